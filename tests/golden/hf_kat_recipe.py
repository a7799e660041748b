"""Recipe shared by ``make_hf_olmo2_kat.py`` (which runs ``transformers``' own Olmo2 / Olmo models on the CPU and
stores their logits) and by the tests that replay the stored cases: model shapes, the seeded weights under the
Hugging Face parameter names, the token ids and the padding mask.

The weights are not stored: they are drawn from torch's CPU generator in a fixed order, so the fixture holds
only the logits (a changed random stream would show as a failing test, not as silent drift).

The HF models are an implementation of the same architecture that is independent of this repository:
``scripts/convert_olmo2_to_hf.py:110-163`` of the reference maps OLMo checkpoints onto ``Olmo2ForCausalLM`` (fused
``att_proj`` rows = q | k | v, ``ff_proj`` rows = up | gate), so logits of the HF model on converted weights pin
the block composition of ``olmo/model.py:728-823`` (norm placement, full-width QK-norm, split orders).
"""

from __future__ import annotations

from typing import Dict, Optional

import torch

# name -> architecture; head_dim 32 throughout (the smallest the device kernels take)
CASES = {
    # OLMo-2 wiring: post-norm RMS (affine), QK-norm over the full projected width, rope theta 5e5
    "olmo2_mha": dict(arch="olmo2", d=128, heads=4, kv_heads=4, layers=3, ffn=192, vocab=96, theta=500000.0, eps=1e-6),
    "olmo2_gqa": dict(arch="olmo2", d=128, heads=4, kv_heads=2, layers=3, ffn=192, vocab=96, theta=500000.0, eps=1e-6),
    # OLMo-1 wiring: pre-norm, non-parametric LayerNorm (eps 1e-5), rope theta 1e4, optional clip_qkv
    "olmo1": dict(arch="olmo", d=128, heads=4, kv_heads=4, layers=3, ffn=192, vocab=96, theta=10000.0, eps=1e-5),
    "olmo1_clip": dict(arch="olmo", d=128, heads=4, kv_heads=4, layers=3, ffn=192, vocab=96, theta=10000.0, eps=1e-5,
                       clip_qkv=0.3),
}
SEQ = 24
BATCH = 3
LEFT_PAD = (0, 5, 11)  # padded positions at the start of each row


def hf_state_dict(case: dict, seed: int) -> Dict[str, torch.Tensor]:
    """fp32 weights under ``transformers``' parameter names; Linear / embedding ~ N(0, 0.08) (large enough that a
    wiring mistake moves the logits by far more than the tolerance), norm weights ~ N(1, 0.2)."""
    g = torch.Generator().manual_seed(seed)
    d, hd = case["d"], case["d"] // case["heads"]
    dkv, f, V = hd * case["kv_heads"], case["ffn"], case["vocab"]

    def lin(n, k):
        return torch.randn(n, k, generator=g) * 0.08

    def nw(n):
        return 1.0 + 0.2 * torch.randn(n, generator=g)

    sd: Dict[str, torch.Tensor] = {"model.embed_tokens.weight": lin(V, d)}
    for i in range(case["layers"]):
        p = f"model.layers.{i}."
        sd[p + "self_attn.q_proj.weight"] = lin(d, d)
        sd[p + "self_attn.k_proj.weight"] = lin(dkv, d)
        sd[p + "self_attn.v_proj.weight"] = lin(dkv, d)
        sd[p + "self_attn.o_proj.weight"] = lin(d, d)
        sd[p + "mlp.gate_proj.weight"] = lin(f, d)
        sd[p + "mlp.up_proj.weight"] = lin(f, d)
        sd[p + "mlp.down_proj.weight"] = lin(d, f)
        if case["arch"] == "olmo2":
            sd[p + "self_attn.q_norm.weight"] = nw(d)
            sd[p + "self_attn.k_norm.weight"] = nw(dkv)
            sd[p + "post_attention_layernorm.weight"] = nw(d)
            sd[p + "post_feedforward_layernorm.weight"] = nw(d)
    if case["arch"] == "olmo2":
        sd["model.norm.weight"] = nw(d)
    sd["lm_head.weight"] = lin(V, d)
    return sd


def inputs(case: dict, seed: int):
    """Token ids ``[BATCH, SEQ]`` and a left-padding mask (1 = real token)."""
    g = torch.Generator().manual_seed(seed + 1000)
    ids = torch.randint(0, case["vocab"], (BATCH, SEQ), generator=g)
    mask = torch.ones(BATCH, SEQ, dtype=torch.int64)
    for b, n in enumerate(LEFT_PAD):
        mask[b, :n] = 0
    return ids, mask


def model_config(case: dict):
    """The case as this repository's ``ModelConfig`` (reference field names, ``olmo/config.py:235-497``)."""
    from olmo_amd.config import ModelConfig

    olmo2 = case["arch"] == "olmo2"
    return ModelConfig(
        d_model=case["d"], n_heads=case["heads"], n_kv_heads=case["kv_heads"], n_layers=case["layers"],
        mlp_hidden_size=2 * case["ffn"], rope=True, alibi=False, include_bias=False, weight_tying=False,
        vocab_size=case["vocab"], embedding_size=case["vocab"], max_sequence_length=64,
        layer_norm_type="rms" if olmo2 else "default", layer_norm_with_affine=olmo2, layer_norm_eps=case["eps"],
        attention_layer_norm=olmo2, norm_after=olmo2, rope_theta=case["theta"], clip_qkv=case.get("clip_qkv"),
        attention_dropout=0.0, residual_dropout=0.0, embedding_dropout=0.0)


def to_olmo_state_dict(case: dict, sd: Dict[str, torch.Tensor], swap_up_gate: bool = False,
                       swap_norms: bool = False) -> Dict[str, torch.Tensor]:
    """HF names -> the reference's names.  OLMo-2 goes through the product's own converter (so the converter is
    checked against an independent model as well); OLMo-1 has no norm weights and is fused here.
    ``swap_*`` build deliberately wrong wirings for the negative tests."""
    from olmo_amd.checkpoint import hf_olmo2_to_olmo_state_dict

    cfg = model_config(case)
    if case["arch"] == "olmo2":
        out = hf_olmo2_to_olmo_state_dict(sd, cfg)
    else:
        out = {}
        for i in range(case["layers"]):
            s, t = f"model.layers.{i}.", f"transformer.blocks.{i}."
            out[t + "att_proj.weight"] = torch.cat([sd[s + f"self_attn.{p}_proj.weight"] for p in "qkv"], dim=0)
            out[t + "ff_proj.weight"] = torch.cat([sd[s + "mlp.up_proj.weight"], sd[s + "mlp.gate_proj.weight"]], dim=0)
            out[t + "attn_out.weight"] = sd[s + "self_attn.o_proj.weight"]
            out[t + "ff_out.weight"] = sd[s + "mlp.down_proj.weight"]
        out["transformer.wte.weight"] = sd["model.embed_tokens.weight"]
        out["transformer.ff_out.weight"] = sd["lm_head.weight"]
    if swap_up_gate:
        for i in range(case["layers"]):
            k = f"transformer.blocks.{i}.ff_proj.weight"
            up, gate = out[k].chunk(2, dim=0)
            out[k] = torch.cat([gate, up], dim=0)
    if swap_norms:
        for i in range(case["layers"]):
            a, b = f"transformer.blocks.{i}.attn_norm.weight", f"transformer.blocks.{i}.ff_norm.weight"
            out[a], out[b] = out[b], out[a]
    return out


def seed_of(name: str) -> int:
    return 100 + sorted(CASES).index(name)


def hf_model(case: dict, sd: Optional[Dict[str, torch.Tensor]] = None):
    """The ``transformers`` model of a case (CPU, fp32, eager attention), weights loaded strictly."""
    import transformers

    common = dict(vocab_size=case["vocab"], hidden_size=case["d"], intermediate_size=case["ffn"],
                  num_hidden_layers=case["layers"], num_attention_heads=case["heads"],
                  num_key_value_heads=case["kv_heads"], max_position_embeddings=64, rope_theta=case["theta"],
                  tie_word_embeddings=False, pad_token_id=None, attention_bias=False, attention_dropout=0.0)
    if case["arch"] == "olmo2":
        cfg = transformers.Olmo2Config(rms_norm_eps=case["eps"], **common)
        m = transformers.Olmo2ForCausalLM(cfg)
    else:
        cfg = transformers.OlmoConfig(clip_qkv=case.get("clip_qkv"), **common)
        m = transformers.OlmoForCausalLM(cfg)
    m = m.to(torch.float32).eval()
    if sd is not None:
        missing, unexpected = m.load_state_dict(sd, strict=False)
        assert not unexpected and all("rotary" in k or "inv_freq" in k for k in missing), (missing, unexpected)
    return m
