"""The HF surface (``olmo_amd/hf.py``) under transformers' own ``generate`` (``hf_olmo/modeling_olmo.py:41-261``).

CPU part: ``OLMoForCausalLM`` wrapped around a stand-in core that computes with the oracle and keeps its keys and
values in the product's ``KVCache`` buffers, so that the wrapper's ``forward`` / ``prepare_inputs_for_generation`` /
``OLMoCache`` are driven by ``GenerationMixin.generate`` without a GPU.  What they must produce is fixed by an
implementation this repository did not write: ``transformers.Olmo2ForCausalLM`` / ``OlmoForCausalLM`` on the same
seeded weights (``tests/golden/hf_kat_recipe.py``), run through the same ``generate`` call -- greedy, left-padded,
and transformers' beam search (which reorders the cache rows after every step).

GPU part: the same comparison with the real model (HIP kernels, fp32) inside the wrapper.
"""
import pytest
import torch
import torch.nn as nn

transformers = pytest.importorskip("transformers")

from olmo_amd import hf as H  # noqa: E402
from olmo_amd.model import KVCache, LayerKV, OLMoOutput  # noqa: E402
from oracle import model as om  # noqa: E402
from tests.golden import hf_kat_recipe as R  # noqa: E402


class OracleCore(nn.Module):
    """Stands in for ``olmo_amd.model.OLMo`` on the CPU: same ``forward`` arguments and ``OLMoOutput``, the cache in
    ``KVCache`` buffers (here with the keys in the reference's un-rotated form, which only this class reads)."""

    def __init__(self, cfg, weights, capacity=64):
        super().__init__()
        self.config, self.capacity = cfg, capacity
        self.oracle = om.OracleModel(cfg, weights, torch.float32)
        self.transformer = nn.ModuleDict({"wte": nn.Embedding.from_pretrained(weights["transformer.wte.weight"])})
        self.calls = []

    def forward(self, input_ids, input_embeddings=None, attention_mask=None, attention_bias=None, past_key_values=None,
                use_cache=False, last_logits_only=False, output_hidden_states=None):
        assert input_embeddings is None and attention_bias is None
        c = self.config
        B, T = input_ids.shape
        cache, past = None, None
        if past_key_values:
            assert isinstance(past_key_values[0], LayerKV), "the wrapper hands back the product's own views"
            cache = past_key_values[0].cache
            past = [(k, v) for k, v in past_key_values]
        self.calls.append((T, 0 if cache is None else cache.length))
        logits, kvs = self.oracle.forward(input_ids, attention_mask=attention_mask, past_key_values=past, use_cache=use_cache)
        if not use_cache:
            return OLMoOutput(logits, None, None)
        if cache is None:
            cache = KVCache(c.n_layers, B, c.effective_n_kv_heads, self.capacity, c.d_model // c.n_heads, torch.float32, "cpu")
        L0 = cache.length
        for i, (k, v) in enumerate(kvs):
            cache.k[i][:, :, L0:L0 + T] = k[:, :, L0:]
            cache.v[i][:, :, L0:L0 + T] = v[:, :, L0:]
        cache.set_length(L0 + T)
        return OLMoOutput(logits, cache.views(), None)


def wrapped(name):
    case, seed = R.CASES[name], R.seed_of(name)
    sd = R.hf_state_dict(case, seed)
    cfg = R.model_config(case)
    cfg.eos_token_id, cfg.pad_token_id = case["vocab"] - 1, case["vocab"] - 1
    core = OracleCore(cfg, R.to_olmo_state_dict(case, sd))
    ours = H.OLMoForCausalLM(H.OLMoConfig.from_model_config(cfg, use_cache=True), model=core)
    theirs = R.hf_model(case, sd)
    theirs.generation_config.pad_token_id = cfg.pad_token_id
    theirs.generation_config.eos_token_id = None  # fixed length on both sides
    return case, seed, ours, theirs, core


def test_is_a_transformers_model_and_registered():
    assert issubclass(H.OLMoForCausalLM, transformers.PreTrainedModel)
    assert issubclass(H.OLMoForCausalLM, transformers.GenerationMixin)
    assert issubclass(H.OLMoConfig, transformers.PretrainedConfig)
    cfg = transformers.AutoConfig.for_model("hf_olmo", d_model=128, n_heads=4)  # configuration_olmo.py:63
    assert isinstance(cfg, H.OLMoConfig) and cfg.hidden_size == 128 and cfg.num_attention_heads == 4
    assert cfg.use_cache is False and cfg.architectures == ["OLMoForCausalLM"]
    from transformers.models.auto.modeling_auto import MODEL_FOR_CAUSAL_LM_MAPPING

    assert MODEL_FOR_CAUSAL_LM_MAPPING[H.OLMoConfig] is H.OLMoForCausalLM  # modeling_olmo.py:261
    assert H.OLMoForCausalLM.can_generate() and H.OLMoForCausalLM._no_split_modules == ["OLMoBlock"]


def test_config_save_and_load(tmp_path):
    """``tests/hf_olmo/configuration_olmo_test.py:6-19``: ``save_pretrained`` / ``from_pretrained`` keep every
    ``ModelConfig`` field, a non-default one included."""
    from dataclasses import asdict

    from olmo_amd.config import ModelConfig

    mc = ModelConfig(d_model=128, n_heads=4, rope=True, rope_theta=500000, clip_qkv=8.0)
    d = asdict(mc)
    d.pop("extra", None)
    cfg = H.OLMoConfig(**d)
    cfg.save_pretrained(tmp_path)
    loaded = H.OLMoConfig.from_pretrained(tmp_path)
    assert cfg.to_dict() == loaded.to_dict()
    for k, v in d.items():
        assert getattr(loaded, k) == v, k
    assert loaded.to_model_config() == mc and loaded.model_type == "hf_olmo"


@pytest.mark.parametrize("name", ["olmo2_gqa", "olmo1_clip"])
def test_transformers_greedy_loop_matches_independent_model(name):
    case, seed, ours, theirs, core = wrapped(name)
    ids, _ = R.inputs(case, seed)
    ids = ids[:, :10]
    kw = dict(max_new_tokens=12, do_sample=False, eos_token_id=None)
    want = theirs.generate(ids, attention_mask=torch.ones_like(ids), **kw)
    got = ours.generate(ids, attention_mask=torch.ones_like(ids), loop="transformers", **kw)
    assert torch.equal(got, want)
    # one prefill of the prompt, then one token per call against the growing cache
    assert core.calls[0] == (10, 0) and core.calls[1:] == [(1, 10 + i) for i in range(11)]


def test_transformers_greedy_loop_left_padded():
    case, seed, ours, theirs, _ = wrapped("olmo2_mha")
    ids, mask = R.inputs(case, seed)
    ids, mask = ids[:, :16], mask[:, :16]
    kw = dict(max_new_tokens=8, do_sample=False, eos_token_id=None)
    want = theirs.generate(ids, attention_mask=mask, **kw)
    got = ours.generate(ids, attention_mask=mask, loop="transformers", **kw)
    assert torch.equal(got, want)


def test_transformers_beam_search_reorders_the_buffers():
    case, seed, ours, theirs, _ = wrapped("olmo2_gqa")
    ids, _ = R.inputs(case, seed)
    ids = ids[:2, :8]
    kw = dict(max_new_tokens=10, num_beams=3, do_sample=False, eos_token_id=None, length_penalty=1.0, early_stopping=False)
    want = theirs.generate(ids, attention_mask=torch.ones_like(ids), **kw)
    got = ours.generate(ids, attention_mask=torch.ones_like(ids), loop="transformers", **kw)
    assert torch.equal(got, want)


def test_forward_cache_forms():
    """A list in, a list out (as the reference); a ``Cache`` in, an :class:`OLMoCache` out that continues in place;
    a populated foreign ``DynamicCache`` is taken over as per-layer ``(k, v)``."""
    case, seed, ours, theirs, core = wrapped("olmo2_mha")
    ids, _ = R.inputs(case, seed)
    full = ours(ids[:, :12]).logits
    out = ours(ids[:, :8], use_cache=True)
    assert isinstance(out.past_key_values, list) and isinstance(out.past_key_values[0], LayerKV)
    out2 = ours(ids[:, 8:12], past_key_values=out.past_key_values, use_cache=True)
    assert (out2.logits - full[:, 8:12]).abs().max() < 1e-5
    out = ours(ids[:, :8], past_key_values=transformers.DynamicCache(), use_cache=True)
    c = out.past_key_values
    assert isinstance(c, H.OLMoCache) and isinstance(c, transformers.Cache) and c.get_seq_length() == 8
    assert len(c) == case["layers"] and c.layers[0].keys.shape[-2] == 8
    out2 = ours(ids[:, 8:12], past_key_values=c, use_cache=True)
    assert out2.past_key_values is c and c.get_seq_length() == 12 and c.layers[1].values.shape[-2] == 12
    assert (out2.logits - full[:, 8:12]).abs().max() < 1e-5
    c.crop(-4)
    assert c.get_seq_length() == 8 and c.layers[0].keys.shape[-2] == 8
    out3 = ours(ids[:, 8:12], past_key_values=c, use_cache=True)
    assert (out3.logits - full[:, 8:12]).abs().max() < 1e-5
    c.batch_select_indices(torch.tensor([2, 0]))
    assert c.kv.B == 2 and c.get_seq_length() == 12
    out4 = ours(ids[[2, 0], 12:13], past_key_values=c, use_cache=True)
    assert (out4.logits - ours(ids[[2, 0], :13]).logits[:, 12:13]).abs().max() < 1e-5
    with pytest.raises(ValueError, match="output_attentions"):
        ours(ids, output_attentions=True)


def test_prepare_inputs_for_generation():
    case, seed, ours, _, _ = wrapped("olmo1")
    ids, _ = R.inputs(case, seed)
    inp = ours.prepare_inputs_for_generation(ids, past_key_values=None, attention_mask=None)
    assert inp["input_ids"].shape == ids.shape and inp["use_cache"] is True
    out = ours(ids[:, :8], use_cache=True)
    inp = ours.prepare_inputs_for_generation(ids[:, :9], past_key_values=out.past_key_values, use_cache=True,
                                             position_ids="dropped")
    assert inp["input_ids"].shape == (ids.shape[0], 1) and "position_ids" not in inp
    inp = ours.prepare_inputs_for_generation(ids[:, :11], past_key_values=out.past_key_values, next_sequence_length=3)
    assert torch.equal(inp["input_ids"], ids[:, 8:11]) and "next_sequence_length" not in inp


def test_default_loop_is_the_captured_one_only_where_it_decodes_as_transformers_would():
    """A ``generate`` call that names no loop: plain greedy decoding of a stated number of tokens goes to the captured
    loop with the end and padding tokens of ``generation_config`` filled in; sampling, beams, a default length, several
    end tokens or any argument the captured loop does not know go to transformers' loop."""
    case, seed, ours, _, _ = wrapped("olmo1")
    ids, _ = R.inputs(case, seed)
    gc = ours.generation_config
    gc.eos_token_id, gc.pad_token_id = 7, 3
    loop, kw = ours._route(ids, (), dict(max_new_tokens=4))
    assert loop == "captured" and kw["eos_token_id"] == 7 and kw["pad_token_id"] == 3
    loop, kw = ours._route(ids, (), dict(max_new_tokens=4, eos_token_id=None, pad_token_id=9))
    assert loop == "captured" and kw["eos_token_id"] is None and kw["pad_token_id"] == 9
    gc.eos_token_id = [7]
    assert ours._route(ids, (), dict(max_new_tokens=4))[1]["eos_token_id"] == 7
    gc.eos_token_id = [7, 8]
    assert ours._route(ids, (), dict(max_new_tokens=4))[0] == "transformers"
    gc.eos_token_id = 7
    for kw in (dict(), dict(max_new_tokens=4, do_sample=True), dict(max_new_tokens=4, num_beams=2),
               dict(max_new_tokens=4, repetition_penalty=1.1), dict(max_length=30)):
        assert ours._route(ids, (), kw)[0] == "transformers", kw
    gc.do_sample = True
    assert ours._route(ids, (), dict(max_new_tokens=4))[0] == "transformers"
    gc.do_sample = False
    assert ours._route(None, (), dict(max_new_tokens=4))[0] == "transformers"
    # on the CPU model of this file the default route must therefore be runnable for a sampled call: transformers' loop
    gc.eos_token_id = None
    out = ours.generate(ids[:, :6], attention_mask=torch.ones_like(ids[:, :6]), max_new_tokens=3, do_sample=True, top_k=5)
    assert out.shape == (ids.shape[0], 9)


def test_captured_loop_rejects_what_it_does_not_know():
    case, seed, ours, _, _ = wrapped("olmo1")
    ids, _ = R.inputs(case, seed)
    with pytest.raises(TypeError, match="repetition_penalty"):
        ours.generate(ids, loop="captured", repetition_penalty=1.2)
    with pytest.raises(ValueError, match="loop"):
        ours.generate(ids, loop="other")


# ---- GPU: the real model inside the wrapper ------------------------------------------------------------------
def _gpu_wrapped(name):
    from olmo_amd.model import OLMo

    case, seed = R.CASES[name], R.seed_of(name)
    sd = R.hf_state_dict(case, seed)
    cfg = R.model_config(case)
    cfg.eos_token_id, cfg.pad_token_id = case["vocab"] - 1, case["vocab"] - 1
    model = OLMo(cfg, device="cuda", dtype=torch.float32, max_cache_len=64)
    model.load_reference_state_dict(R.to_olmo_state_dict(case, sd))
    ours = H.OLMoForCausalLM(H.OLMoConfig.from_model_config(cfg, use_cache=True), model=model)
    theirs = R.hf_model(case, sd)
    theirs.generation_config.pad_token_id = cfg.pad_token_id
    theirs.generation_config.eos_token_id = None
    return case, seed, ours, theirs


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["olmo2_gqa", "olmo1_clip"])
def test_gpu_transformers_loops_match_independent_model_and_captured_loop(name):
    case, seed, ours, theirs = _gpu_wrapped(name)
    ids, mask = R.inputs(case, seed)
    ids, mask = ids[:, :16], mask[:, :16]
    kw = dict(max_new_tokens=12, do_sample=False, eos_token_id=None)
    want = theirs.generate(ids, attention_mask=mask, **kw)
    got = ours.generate(ids.cuda(), attention_mask=mask.cuda(), loop="transformers", **kw)
    assert torch.equal(got.cpu(), want)
    assert ours._route(ids, (), dict(kw, attention_mask=mask))[0] == "captured"
    cap = ours.generate(ids.cuda(), attention_mask=mask.cuda(), **kw)  # no loop named: the captured one
    assert torch.equal(cap.cpu(), want)
    # an end token that does occur, set where HF keeps it (generation_config), named by neither call: both loops stop
    # a sequence there, pad after it and end once every sequence has ended, and give what the independent model gives
    new = want[:, ids.shape[1]:]
    eos = int(new[0, 3])
    for m in (ours, theirs):
        m.generation_config.eos_token_id, m.generation_config.pad_token_id = eos, 0
    want_e = theirs.generate(ids, attention_mask=mask, max_new_tokens=12)
    assert (want_e[0, ids.shape[1]:] == eos).sum() == 1 and (want_e[0, ids.shape[1]:] == 0).any()
    via_hf = ours.generate(ids.cuda(), attention_mask=mask.cuda(), max_new_tokens=12, loop="transformers")
    default = ours.generate(ids.cuda(), attention_mask=mask.cuda(), max_new_tokens=12)
    assert torch.equal(via_hf.cpu(), want_e) and torch.equal(default.cpu(), want_e)
    one = ours.generate(ids[:1].cuda(), attention_mask=mask[:1].cuda(), max_new_tokens=12)  # ends early: cut after the end token
    assert torch.equal(one.cpu(), theirs.generate(ids[:1], attention_mask=mask[:1], max_new_tokens=12))
    assert one.shape[1] < ids.shape[1] + 12
    for m in (ours, theirs):
        m.generation_config.eos_token_id = None
    kw = dict(max_new_tokens=10, num_beams=3, do_sample=False, eos_token_id=None, length_penalty=1.0, early_stopping=False)
    want = theirs.generate(ids[:2, 11:], attention_mask=torch.ones_like(ids[:2, 11:]), **kw)
    got = ours.generate(ids[:2, 11:].cuda(), attention_mask=torch.ones_like(ids[:2, 11:]).cuda(), loop="transformers", **kw)
    assert torch.equal(got.cpu(), want)


@pytest.mark.gpu
def test_gpu_foreign_dynamic_cache_is_taken_over():
    """Keys and values another implementation computed (``transformers.Olmo2ForCausalLM``'s ``DynamicCache``: keys
    normalised and rotated the HF way) cannot be continued blindly; the reference-form list can.  A populated cache of
    the wrapper itself continues in place."""
    case, seed, ours, theirs = _gpu_wrapped("olmo2_mha")
    ids, _ = R.inputs(case, seed)
    ids = ids.cuda()
    full = ours(ids[:, :12]).logits
    out = ours(ids[:, :8], past_key_values=transformers.DynamicCache(), use_cache=True)
    c = out.past_key_values
    assert isinstance(c, H.OLMoCache) and c.get_seq_length() == 8
    out2 = ours(ids[:, 8:12], past_key_values=c, use_cache=True)
    assert out2.past_key_values is c and (out2.logits - full[:, 8:12]).abs().max() < 2e-4
    c.crop(-4)
    c.reorder_cache(torch.tensor([1, 2, 0], device="cuda"))
    out3 = ours(ids[[1, 2, 0], 8:12], past_key_values=c, use_cache=True)
    assert (out3.logits - full[[1, 2, 0], 8:12]).abs().max() < 2e-4


@pytest.mark.gpu
def test_gpu_save_pretrained_from_pretrained(tmp_path):
    """A directory written by ``save_pretrained`` loads back through ``OLMoForCausalLM.from_pretrained`` and through
    ``AutoModelForCausalLM`` (the registration of ``modeling_olmo.py:261``) with identical logits -- what
    ``tests/hf_olmo/modeling_olmo_test.py:9-26`` does with the reference's fixture checkpoint (whose weight file does
    not ship)."""
    from olmo_amd.model import OLMo

    case, seed = R.CASES["olmo2_gqa"], R.seed_of("olmo2_gqa")
    cfg = R.model_config(case)
    model = OLMo(cfg, device="cuda", dtype=torch.float32, max_cache_len=64)
    model.load_reference_state_dict(R.to_olmo_state_dict(case, R.hf_state_dict(case, seed)))
    hf = H.OLMoForCausalLM(H.OLMoConfig.from_model_config(cfg, use_cache=True), model=model)
    ids, _ = R.inputs(case, seed)
    ids = ids.cuda()
    want = hf(ids).logits
    hf.save_pretrained(tmp_path)
    for cls in (H.OLMoForCausalLM, transformers.AutoModelForCausalLM):
        back = cls.from_pretrained(tmp_path, dtype=torch.float32)
        assert isinstance(back, H.OLMoForCausalLM)
        got = back(ids).logits
        assert torch.equal(got, want)
