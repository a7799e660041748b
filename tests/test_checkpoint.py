"""Host-side checkpoint code (no GPU): quantize_config.json, state-dict key fix-ups, OLMo <-> HF Olmo2
tensor layouts."""
import json

import pytest
import torch

from olmo_amd.checkpoint import (BaseQuantizeConfig, hf_olmo2_to_olmo_state_dict, make_state_dict_compatible,
                                 olmo_to_hf_olmo2_state_dict)
from olmo_amd.config import ModelConfig


def test_quantize_config_defaults_validation_and_json(tmp_path):
    # defaults and messages of AGQ/auto_gptq/modeling/_base.py:43-66
    qc = BaseQuantizeConfig()
    assert (qc.bits, qc.group_size, qc.damp_percent, qc.desc_act, qc.static_groups, qc.sym, qc.true_sequential) == \
        (4, -1, 0.01, True, False, True, True)
    with pytest.raises(ValueError, match="only support quantize to"):
        BaseQuantizeConfig(bits=5)
    with pytest.raises(ValueError, match="group_size"):
        BaseQuantizeConfig(group_size=0)
    with pytest.raises(ValueError, match="damp_percent"):
        BaseQuantizeConfig(damp_percent=1.5)
    # the file the reference's quantization driver writes (inference/compression/run_quantization.py:39-43)
    qc = BaseQuantizeConfig(bits=4, group_size=128)
    qc.save_pretrained(str(tmp_path))
    d = json.load(open(tmp_path / "quantize_config.json"))
    assert set(d) == {"bits", "group_size", "damp_percent", "desc_act", "static_groups", "sym", "true_sequential",
                      "model_name_or_path", "model_file_base_name"}
    d["some_future_key"] = 1  # unknown keys in a file are ignored
    json.dump(d, open(tmp_path / "quantize_config.json", "w"))
    assert BaseQuantizeConfig.from_pretrained(str(tmp_path)) == qc


def _cfg():
    return ModelConfig(d_model=8, n_heads=2, n_kv_heads=1, n_layers=2, mlp_hidden_size=12, rope=True, alibi=False,
                       vocab_size=10, embedding_size=16, layer_norm_type="rms", attention_layer_norm=True,
                       norm_after=True, include_bias=False, weight_tying=False)


def test_state_dict_fixups():
    cfg = _cfg()
    sd = {
        "transformer._fsdp_wrapped_module.wte.weight": torch.zeros(1),
        "transformer.blocks.0.norm.weight": torch.arange(3.0),
        "transformer.block_groups.0.0.attn_out.weight": torch.ones(1),
        "transformer.block_groups.0.1.attn_out.weight": 2 * torch.ones(1),
        "transformer.block_groups.1.0.attn_out.weight": 3 * torch.ones(1),
        "transformer.block_groups.1.1.attn_out.weight": 4 * torch.ones(1),
    }
    out = make_state_dict_compatible(sd, cfg)
    assert "transformer.wte.weight" in out
    assert torch.equal(out["transformer.blocks.0.attn_norm.weight"], torch.arange(3.0))
    assert torch.equal(out["transformer.blocks.0.ff_norm.weight"], torch.arange(3.0))
    assert "transformer.blocks.0.norm.weight" not in out
    assert [out[f"transformer.blocks.{i}.attn_out.weight"].item() for i in range(4)] == [1, 2, 3, 4]


def test_hf_olmo2_layout_split_orders_and_round_trip():
    cfg = _cfg()
    d, hd, dkv, h = 8, 4, 4, 12
    sd = {"transformer.wte.weight": torch.randn(16, d), "transformer.ln_f.weight": torch.randn(d),
          "transformer.ff_out.weight": torch.randn(16, d)}
    for i in range(2):
        b = f"transformer.blocks.{i}."
        sd[b + "att_proj.weight"] = torch.arange((d + 2 * dkv) * d, dtype=torch.float32).view(d + 2 * dkv, d) + 1000 * i
        sd[b + "ff_proj.weight"] = torch.arange(h * d, dtype=torch.float32).view(h, d) + 1000 * i
        sd[b + "attn_out.weight"], sd[b + "ff_out.weight"] = torch.randn(d, d), torch.randn(d, h // 2)
        for n in ("attn_norm", "ff_norm", "q_norm"):
            sd[b + n + ".weight"] = torch.randn(d)
        sd[b + "k_norm.weight"] = torch.randn(dkv)
    hf = olmo_to_hf_olmo2_state_dict(sd, cfg)
    # scripts/convert_olmo2_to_hf.py:115-121: rows [0,d) are q, then k, then v; ff_proj chunks are (up, gate)
    w = sd["transformer.blocks.1.att_proj.weight"]
    assert torch.equal(hf["model.layers.1.self_attn.q_proj.weight"], w[:d])
    assert torch.equal(hf["model.layers.1.self_attn.k_proj.weight"], w[d:d + dkv])
    assert torch.equal(hf["model.layers.1.self_attn.v_proj.weight"], w[d + dkv:])
    u = sd["transformer.blocks.0.ff_proj.weight"]
    assert torch.equal(hf["model.layers.0.mlp.up_proj.weight"], u[:h // 2])
    assert torch.equal(hf["model.layers.0.mlp.gate_proj.weight"], u[h // 2:])
    assert torch.equal(hf["model.layers.0.post_attention_layernorm.weight"], sd["transformer.blocks.0.attn_norm.weight"])
    assert torch.equal(hf["model.layers.0.post_feedforward_layernorm.weight"], sd["transformer.blocks.0.ff_norm.weight"])
    assert torch.equal(hf["lm_head.weight"], sd["transformer.ff_out.weight"])
    back = hf_olmo2_to_olmo_state_dict(hf, cfg)
    assert set(back) == set(sd)
    assert all(torch.equal(back[k], sd[k]) for k in sd)
    # tied head: the embedding stands in (convert_olmo2_to_hf.py:160-162)
    sd.pop("transformer.ff_out.weight")
    assert torch.equal(olmo_to_hf_olmo2_state_dict(sd, cfg)["lm_head.weight"], sd["transformer.wte.weight"])


def test_sampler_classes_mirror_reference_arguments():
    from olmo_amd.beam_search import DeterministicSampler, MultinomialSampler, TopKSampler, TopPSampler

    assert DeterministicSampler().greedy
    assert MultinomialSampler(temperature=0.5).params() == {"temperature": 0.5, "top_k": 0, "top_p": 1.0}
    assert TopKSampler().params() == {"temperature": 1.0, "top_k": 1, "top_p": 1.0}  # defaults of olmo/beam_search.py:163-172
    assert TopPSampler().params() == {"temperature": 1.0, "top_k": 0, "top_p": 0.9}  # :217-231
    with pytest.raises(ValueError, match="p must be a positive float no greater than 1.0"):
        TopPSampler(p=1.5)
    with pytest.raises(ValueError, match="k must be a postive integer"):
        TopKSampler(k=0).check(100)
