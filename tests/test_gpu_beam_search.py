"""Beam search on the device: the selection kernels against torch, the search against the known-answer cases of
the reference's own tests (``tests/golden/beam_search_kat.json``), the attention kernel that reads beam histories
through a row table against the plain kernel on caches gathered the reference's way, and ``OLMo.generate`` with
beams against the oracle's search driven by the oracle's forward pass."""
import json
import os
import warnings

import numpy as np
import pytest
import torch

from oracle import beam_search as obs
from tests.test_gpu_model import build_pair, say, small_cfg

pytestmark = pytest.mark.gpu

KAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "beam_search_kat.json")))


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from olmo_amd import _lib

    _lib.lib()
    return torch.device("cuda:0")


@pytest.mark.parametrize("rows,n", [(1, 6), (3, 1000), (4, 100352), (2, 50281)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_log_softmax(dev, rows, n, dtype):
    say("log_softmax", rows, n, dtype)
    from olmo_amd import ops

    x = (torch.randn(rows, n, generator=torch.Generator().manual_seed(n)) * 4).to(dtype)
    got = ops.log_softmax(x.to(dev)).cpu()
    want = torch.log_softmax(x.double(), dim=-1)
    assert got.dtype == torch.float32
    assert (got.double() - want).abs().max().item() < 2e-5  # fp32 arithmetic on values up to ~30
    assert abs(torch.exp(got.double()).sum(-1) - 1).max().item() < 1e-4


@pytest.mark.parametrize("rows,n,k", [(1, 6, 3), (5, 6, 6), (3, 1000, 7), (6, 100352, 4), (2, 4097, 64), (4, 36, 6)])
def test_topk_values_order_and_ties(dev, rows, n, k):
    """Values equal torch's; indices follow the stated tie rule (ascending index among equals), checked against a
    stable descending sort.  The rows hold few distinct values, -inf and the float minimum, so ties are the rule."""
    say("topk", rows, n, k)
    from olmo_amd import ops

    g = torch.Generator().manual_seed(rows * n + k)
    x = torch.randint(-6, 6, (rows, n), generator=g).float() * 0.25
    x[torch.rand(rows, n, generator=g) < 0.1] = -float("inf")
    x[torch.rand(rows, n, generator=g) < 0.1] = torch.finfo(torch.float32).min
    v, i = ops.topk(x.to(dev), k)
    wv, wi = obs.topk_stable(x, k)
    assert torch.equal(v.cpu(), wv) and torch.equal(i.cpu(), wi)
    assert torch.equal(v.cpu(), torch.topk(x, k, dim=-1).values)
    y = torch.randn(rows, n, generator=g)  # all distinct: indices equal torch's too
    v, i = ops.topk(y.to(dev), k)
    tv, ti = torch.topk(y, k, dim=-1)
    assert torch.equal(v.cpu(), tv) and torch.equal(i.cpu(), ti)


def chain_step(matrix):
    def step(last, state, timestep):
        return torch.log(matrix[last]), state
    return step


@pytest.mark.parametrize("case", KAT["cases"], ids=[c["name"] for c in KAT["cases"]])
def test_search_reference_known_answers(dev, case):
    say("beam search known answer", case["name"])
    from olmo_amd.beam_search import (BeamSearch, LengthNormalizedSequenceLogProbabilityScorer,
                                      RepeatedNGramBlockingConstraint)

    m = torch.tensor(KAT["matrices"][case["matrix"]], device=dev)
    scorer = None if "length_penalty" not in case else LengthNormalizedSequenceLogProbabilityScorer(case["length_penalty"])
    cons = [RepeatedNGramBlockingConstraint(case["ngram_size"])] if case.get("ngram_size") else None
    bs = BeamSearch(KAT["end_index"], max_steps=case["max_steps"], beam_size=case["beam_size"],
                    per_node_beam_size=case.get("per_node_beam_size"), min_steps=case.get("min_steps"),
                    final_sequence_scorer=scorer, constraints=cons)
    start = torch.full((case["batch_size"],), KAT["start_token"], device=dev)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore", RuntimeWarning)
        top, scores = bs.search(start, {}, chain_step(m))
    assert list(top.shape[:2]) == [case["batch_size"], case["beam_size"]]
    np.testing.assert_array_equal(top[0].cpu().numpy(), np.array(case["expected_top_k"]))
    expected = np.log(np.array(case["expected_probs"]))
    if "length_norm" in case:
        expected = expected / np.array(case["length_norm"])
    np.testing.assert_allclose(scores[0].cpu().numpy(), expected, rtol=KAT["rtol"])
    # every batch element started the same way
    assert all(torch.equal(top[b], top[0]) for b in range(top.shape[0]))


def test_search_argument_checks_state_and_warnings(dev):
    """``tests/beam_search_test.py:149-180`` (a tensor in the state is expanded per beam and follows the
    backpointers), ``:289-297`` (per-node width above the number of classes), ``:299-318`` (warnings), and a
    two-argument step function (``:146``)."""
    say("beam search state / checks")
    from olmo_amd.beam_search import BeamSearch, TopPSampler

    m = torch.tensor(KAT["matrices"]["T"], device=dev)
    state = {"foo": torch.tensor([[1, 0, 1], [2, 0, 1], [0, 0, 1], [1, 1, 1], [0, 0, 0]], device=dev)}
    want = state["foo"].repeat_interleave(3, dim=0)
    BeamSearch(5, max_steps=10, beam_size=3).search(torch.zeros(5, dtype=torch.long, device=dev), state,
                                                   lambda last, st: (torch.log(m[last]), st))
    assert torch.equal(state["foo"], want)
    with pytest.raises(ValueError):
        BeamSearch(5, beam_size=20).search(torch.zeros(5, dtype=torch.long, device=dev), {}, chain_step(m))
    start = torch.tensor([4, 4], device=dev)
    with pytest.warns(RuntimeWarning, match="Negligible log probabilities"):
        BeamSearch(5, max_steps=10, beam_size=3).search(start, {}, chain_step(m))
    with pytest.warns(RuntimeWarning, match="Empty sequences predicted"):
        p, lp = BeamSearch(5, beam_size=1).search(start, {}, chain_step(m))
    assert list(p.shape) == [2, 1, 1] and bool((p == 5).all()) and bool((lp == 0).all())
    for bad in (dict(max_steps=0), dict(beam_size=0), dict(per_node_beam_size=0), dict(min_steps=-1),
                dict(min_steps=11, max_steps=10)):
        with pytest.raises(ValueError):
            BeamSearch(5, **bad)
    with pytest.raises(ValueError):
        TopPSampler(p=1.2)


def test_gumbel_topk_draws_without_replacement(dev):
    """The k largest of Gumbel-perturbed log-probabilities are k draws without replacement: first picks follow p,
    ordered pairs follow p_i p_j / (1 - p_i) (chi-square over 120000 rows, 6 classes, 0.1 % level), a temperature
    reshapes p, impossible entries are never drawn, and (seed, counter) reproduce."""
    say("gumbel top-k")
    from olmo_amd import ops
    from scipy.stats import chi2

    p = torch.tensor([0.35, 0.25, 0.2, 0.1, 0.07, 0.03], dtype=torch.float64)
    rows = 120000
    lp = torch.log(p).float().repeat(rows, 1).to(dev)
    g = ops.gumbel_perturb(lp, 1.0, seed=5, counter=1)
    assert torch.equal(g, ops.gumbel_perturb(lp, 1.0, seed=5, counter=1))
    assert not torch.equal(g, ops.gumbel_perturb(lp, 1.0, seed=5, counter=2))
    idx = ops.topk(g, 2)[1].cpu()
    first = torch.bincount(idx[:, 0], minlength=6).double()
    stat = ((first - rows * p) ** 2 / (rows * p)).sum().item()
    assert stat < chi2.ppf(0.999, 5), stat
    pair = torch.zeros(6, 6, dtype=torch.float64)
    pair.index_put_((idx[:, 0], idx[:, 1]), torch.ones(rows, dtype=torch.float64), accumulate=True)
    want = rows * p[:, None] * p[None, :] / (1 - p[:, None])
    want.fill_diagonal_(0)
    assert pair.diag().sum() == 0
    off = want > 0
    stat = ((pair[off] - want[off]) ** 2 / want[off]).sum().item()
    assert stat < chi2.ppf(0.999, 29), stat
    # temperature 2: weights p^(1/2)
    q = p.sqrt() / p.sqrt().sum()
    t = torch.bincount(ops.topk(ops.gumbel_perturb(lp, 0.5, seed=9, counter=3), 1)[1].cpu()[:, 0], minlength=6).double()
    assert ((t - rows * q) ** 2 / (rows * q)).sum().item() < chi2.ppf(0.999, 5)
    # impossible entries
    lp2 = lp.clone()
    lp2[:, 1] = torch.finfo(torch.float32).min
    lp2[:, 4] = -float("inf")
    i2 = ops.topk(ops.gumbel_perturb(lp2, 1.0, seed=1, counter=1), 4)[1].cpu()
    assert not bool(((i2 == 1) | (i2 == 4)).any())


def test_stochastic_samplers_in_search(dev):
    """``tests/beam_search_test.py:320-384, 417-455``: searches with the multinomial, top-k and top-p samplers
    (shapes, token range, an ended beam only repeats the end token), what each sampler may pick, the argument
    checks, and that a seed reproduces."""
    say("samplers in beam search")
    from olmo_amd.beam_search import BeamSearch, MultinomialSampler, TopKSampler, TopPSampler

    m = torch.tensor(KAT["matrices"]["T"], device=dev)
    start = torch.zeros(5, dtype=torch.long, device=dev)
    for make in (lambda: MultinomialSampler(temperature=0.9), lambda: TopKSampler(k=5, with_replacement=True),
                 lambda: TopPSampler(p=0.8), lambda: TopKSampler(k=3, temperature=0.7), lambda: TopPSampler(p=0.5, with_replacement=True)):
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", RuntimeWarning)
            top, lp = BeamSearch(5, beam_size=3, max_steps=10, sampler=make()).search(start, {}, chain_step(m))
            top2, lp2 = BeamSearch(5, beam_size=3, max_steps=10, sampler=make()).search(start, {}, chain_step(m))
        assert list(top.shape[:2]) == [5, 3] and list(lp.shape) == [5, 3]
        assert bool(((0 <= top) & (top <= 5)).all())
        assert torch.equal(top, top2) and torch.equal(lp, lp2)  # same seed, same draws
        ended = torch.cumsum((top == 5).long(), dim=2) > 0
        assert bool((top[ended] == 5).all())
    lps = torch.log(torch.tensor([[0.1, 0.3, 0.3, 0.3, 0.0, 0.0], [0.0, 0.0, 0.4, 0.3, 0.2, 0.1]])).to(dev)  # :66
    for rep in range(20):
        s = MultinomialSampler(temperature=0.9, seed=rep)
        pr, cl, _ = s.sample_nodes(lps, 3, {})
        assert pr.shape == cl.shape == (2, 3) and bool((cl[0] < 4).all()) and bool((cl[1] > 1).all())
        assert torch.equal(pr, lps.gather(1, cl))
        pr, cl, _ = TopKSampler(k=3, temperature=0.9, seed=rep).sample_nodes(lps, 3, {})
        assert bool(((cl[0] > 0) & (cl[0] < 4)).all()) and bool(((cl[1] > 1) & (cl[1] < 5)).all())
        pr, cl, _ = TopPSampler(p=0.8, temperature=0.9, seed=rep).sample_nodes(lps, 3, {})
        assert bool(((cl[0] > 0) & (cl[0] < 4)).all()) and bool(((cl[1] > 1) & (cl[1] < 5)).all())
        pr, cl, _ = TopPSampler(p=0.7, temperature=1.0, with_replacement=True, seed=rep).sample_nodes(lps, 3, {})
        assert bool(((cl[0] >= 1) & (cl[0] <= 3)).all()) and bool(((cl[1] == 2) | (cl[1] == 3)).all())
    for k in (-1, 0, 7):
        with pytest.raises(ValueError):
            BeamSearch(5, beam_size=3, max_steps=10, sampler=TopKSampler(k=k, with_replacement=True)).search(
                start, {}, chain_step(m))


def test_gumbel_sampler_stochastic_beam_search(dev):
    """``GumbelSampler``: (a) ``gumbel_with_max`` puts each row's maximum exactly at the given value and leaves the
    arg-max distributed as the softmax; (b) the reference's own checks (``tests/beam_search_test.py:386-415, 457-472``:
    shapes, ranges, beams ordered by log-probability, ended beams repeat the end token); (c) what the algorithm is
    for: the two sequences a two-step search keeps are a sample without replacement from the joint sequence
    distribution, so a sequence s is kept with probability q_s + sum_r q_r q_s / (1 - q_r) -- checked on 40000
    independent batch rows against the exact figures for all nine sequences of a three-token chain."""
    say("gumbel sampler")
    from olmo_amd import ops
    from olmo_amd.beam_search import BeamSearch, GumbelSampler
    from scipy.stats import chi2

    p = torch.tensor([0.4, 0.3, 0.15, 0.1, 0.05], dtype=torch.float64)
    rows = 60000
    phi = torch.log(p).float().repeat(rows, 1).to(dev)
    t = torch.linspace(-3, 2, rows).to(dev)
    g = ops.gumbel_with_max(phi, t, seed=2, counter=1)
    assert (g.max(dim=1).values - t).abs().max().item() < 1e-5
    am = torch.bincount(g.argmax(dim=1).cpu(), minlength=5).double()
    assert ((am - rows * p) ** 2 / (rows * p)).sum().item() < chi2.ppf(0.999, 4)

    m = torch.tensor(KAT["matrices"]["T"], device=dev)
    top, lp = BeamSearch(5, beam_size=3, max_steps=10, sampler=GumbelSampler()).search(
        torch.zeros(5, dtype=torch.long, device=dev), {}, chain_step(m))
    assert list(top.shape[:2]) == [5, 3] and list(lp.shape) == [5, 3] and bool(((0 <= top) & (top <= 5)).all())
    ended = torch.cumsum((top == 5).long(), dim=2) > 0
    assert bool((top[ended] == 5).all())
    lps = torch.log(torch.tensor([[0.1, 0.3, 0.3, 0.3, 0.0, 0.0], [0.0, 0.0, 0.4, 0.3, 0.2, 0.1]])).to(dev)
    smp = GumbelSampler(seed=4)
    st = smp.init_state(lps, 2, 6)
    lp_b, idx, st = smp.sample_beams(lps, 3, st)
    assert lp_b.shape == idx.shape == (2, 3) and bool((lp_b[:, :-1] >= lp_b[:, 1:]).all())
    assert bool((idx[0] < 4).all()) and bool((idx[1] > 1).all())
    assert st["G_phi_S"].shape == (6,) and st["phi_S"].shape == (6,)

    tr = torch.tensor([[0.5, 0.3, 0.2, 0.0], [0.2, 0.2, 0.6, 0.0], [0.1, 0.7, 0.2, 0.0], [0.3, 0.3, 0.4, 0.0]],
                      dtype=torch.float64)  # rows: last token 0..2 (and an unused end row); the end token never occurs
    q = {(a, b): (tr[0, a] * tr[a, b]).item() for a in range(3) for b in range(3)}
    batch = 40000
    top, _ = BeamSearch(3, beam_size=2, max_steps=2, sampler=GumbelSampler(seed=11)).search(
        torch.zeros(batch, dtype=torch.long, device=dev), {}, chain_step(tr.float().to(dev)))
    codes = (top[:, :, 0] * 3 + top[:, :, 1]).cpu()
    assert bool((codes[:, 0] != codes[:, 1]).all())  # without replacement
    worst = 0.0
    for (a, b), qs in q.items():
        want = qs + sum(qr * qs / (1 - qr) for r, qr in q.items() if r != (a, b))
        got = (codes == a * 3 + b).any(dim=1).double().mean().item()
        sigma = (want * (1 - want) / batch) ** 0.5
        worst = max(worst, abs(got - want) / sigma)
    assert worst < 4.5, worst


@pytest.mark.parametrize("dtype,hd", [(torch.bfloat16, 128), (torch.float32, 32), (torch.bfloat16, 64), (torch.float16, 64)])
def test_attn_decode_beam_equals_gathered_caches(dev, dtype, hd):
    """The row table must give what the reference's per-step cache gather gives: the plain kernel on caches
    materialised row by row from (prompt of the first beam, generated rows by table) -- bit for bit."""
    say("attn_decode_beam", dtype, hd)
    from olmo_amd import ops

    g = torch.Generator().manual_seed(hd)
    B, beam, H, Hkv, P, S = 2, 3, 4, 2, 150, 40
    R, cap, t = B * beam, P + S, 23  # t generated tokens in the cache, the newest at position P + t - 1
    kc = torch.randn(R, Hkv, cap, hd, generator=g).to(dtype).to(dev)
    vc = torch.randn(R, Hkv, cap, hd, generator=g).to(dtype).to(dev)
    q = torch.randn(R, H * hd, generator=g).to(dtype).to(dev)
    src = torch.empty(R, S, dtype=torch.int32)
    for b in range(R):  # any row of the same sequence may hold a step; entries past t stay valid rows
        lo = (b // beam) * beam
        src[b] = torch.randint(lo, lo + beam, (S,), generator=g)
    src = src.to(dev)
    L = P + t
    ws = ops.attn_decode_workspace(R, H, hd, cap, dev)
    bias = torch.zeros(R, cap, device=dev)
    bias[1, 3:9] = torch.finfo(torch.float32).min
    got = ops.attn_decode(q, kc, vc, ws, R, H, Hkv, hd, L - 1, cap, key_bias=bias, beam_src=src, prompt_len=P, beam=beam)
    gk, gv = torch.empty_like(kc), torch.empty_like(vc)
    for b in range(R):
        first = (b // beam) * beam
        gk[b, :, :P], gv[b, :, :P] = kc[first, :, :P], vc[first, :, :P]
        for i in range(S):
            gk[b, :, P + i], gv[b, :, P + i] = kc[src[b, i], :, P + i], vc[src[b, i], :, P + i]
    want = ops.attn_decode(q, gk, gv, ws, R, H, Hkv, hd, L - 1, cap, key_bias=bias)
    assert torch.equal(got, want)
    pos = torch.tensor([L - 1], dtype=torch.int32, device=dev)  # position from device memory
    got2 = ops.attn_decode(q, kc, vc, ws, R, H, Hkv, hd, 0, cap, key_bias=bias, past_len_dev=pos, beam_src=src,
                           prompt_len=P, beam=beam)
    assert torch.equal(got2, want)


def oracle_generate(oracle, ids, mask, eos, **kw):
    """The reference's step function (``olmo/model.py:1677-1714``) over the oracle's forward pass; the state is the
    cache in the reference's form, gathered along the batch axis by the oracle's search."""
    n_layers = oracle.cfg.n_layers

    def step(last, state, timestep):
        if timestep == 0:
            logits, kvs = oracle.forward(ids, attention_mask=mask, use_cache=True, last_logits_only=True)
            st = {}
        else:
            past = [(state[f"k{i}"], state[f"v{i}"]) for i in range(n_layers)]
            am = None
            if mask is not None:
                am = torch.cat([state["mask"], torch.ones(last.shape[0], 1, dtype=state["mask"].dtype)], dim=1)
            logits, kvs = oracle.forward(last.unsqueeze(1), attention_mask=am, past_key_values=past, use_cache=True,
                                         last_logits_only=True)
            st = {}
            if am is not None:
                st["mask"] = am
        if timestep == 0 and mask is not None:
            st["mask"] = mask
        for i, (k, v) in enumerate(kvs):
            st[f"k{i}"], st[f"v{i}"] = k, v
        return torch.log_softmax(logits[:, -1].float(), dim=-1), st

    return obs.beam_search(step, torch.zeros(ids.shape[0], dtype=torch.long), {}, eos, **kw)


@pytest.mark.parametrize("kind,masked", [("ln", False), ("ln", True), ("ln-tied-clip", False)])
def test_generate_with_beams_against_oracle_fp32(dev, kind, masked):
    """fp32 model: same sequences as the oracle's search over the oracle's forward pass, scores within fp32
    noise; with and without left padding, with n-gram blocking, ``min_steps`` and length normalisation."""
    say("generate with beams vs oracle", kind, masked)
    from olmo_amd.beam_search import LengthNormalizedSequenceLogProbabilityScorer, RepeatedNGramBlockingConstraint

    cfg = small_cfg(kind)
    cfg.eos_token_id = 7
    model, oracle = build_pair(cfg, torch.float32, dev, seed=5)
    g = torch.Generator().manual_seed(2)
    ids = torch.randint(8, cfg.vocab_size, (3, 11), generator=g)
    mask = None
    if masked:
        mask = torch.ones(3, 11)
        mask[1, :4] = 0
        mask[2, :1] = 0
    for kw in (dict(beam_size=4, max_steps=9),
               dict(beam_size=3, per_node_beam_size=2, max_steps=7, min_steps=3),
               dict(beam_size=2, max_steps=8, ngram_size=2, length_penalty=0.7),
               dict(beam_size=1, max_steps=5, min_steps=2)):
        okw = dict(kw)
        dkw = dict(kw)
        if "ngram_size" in dkw:
            dkw["constraints"] = [RepeatedNGramBlockingConstraint(dkw.pop("ngram_size"))]
        if "length_penalty" in dkw:
            dkw["final_sequence_scorer"] = LengthNormalizedSequenceLogProbabilityScorer(dkw.pop("length_penalty"))
        out = model.generate(ids.to(dev), attention_mask=None if mask is None else mask.to(dev), **dkw)
        want_t, want_s = oracle_generate(oracle, ids, mask, cfg.eos_token_id, **okw)
        assert out.token_ids.shape == want_t.shape and out.scores.shape == want_s.shape
        assert torch.equal(out.token_ids.cpu(), want_t), (kw, out.token_ids.cpu(), want_t)
        assert (out.scores.cpu() - want_s).abs().max().item() < 2e-3, kw


def test_greedy_generate_end_token_semantics_fp32(dev):
    """The captured greedy loop follows the search's rules for the end token (``olmo/beam_search.py:918-957``): a
    sequence that emitted it only repeats it at no cost, and the result is as long as the longest sequence.  An end
    token is chosen that the model does emit early in one sequence; result against the oracle's search with beam 1
    and against this build's own search."""
    say("greedy end-token semantics")
    cfg = small_cfg("ln")
    model, oracle = build_pair(cfg, torch.float32, dev, seed=5)
    ids = torch.randint(8, cfg.vocab_size, (3, 11), generator=torch.Generator().manual_seed(2))
    free = model.generate(ids.to(dev), max_steps=20, stop_at_eos=False).token_ids[:, 0].cpu()
    assert free.shape == (3, 20)
    for eos in (int(free[0, 2]), int(free[1, 0])):
        cfg.eos_token_id = eos
        out = model.generate(ids.to(dev), max_steps=20)
        want_t, want_s = oracle_generate(oracle, ids, None, eos, beam_size=1, max_steps=20)
        assert torch.equal(out.token_ids.cpu(), want_t), (eos, out.token_ids.cpu(), want_t)
        assert (out.scores.cpu() - want_s).abs().max().item() < 2e-3
        via = model._generate_beam(ids.to(dev), None, 20, 1, None, None, None, None, None)
        assert torch.equal(via.token_ids, out.token_ids) and (via.scores - out.scores).abs().max().item() < 2e-3
    # every sequence ends at once: the loop stops at its 16-step check and the result is cut to the end token
    cfg.eos_token_id = int(free[0, 0])
    one = model.generate(ids[:1].to(dev), max_steps=40)
    assert one.token_ids.shape == (1, 1, 1) and int(one.token_ids[0, 0, 0]) == cfg.eos_token_id


def test_generate_with_beams_bf16_consistency(dev):
    """bf16 OLMo-2 wiring (QK-norm, GQA off / on).  Every returned sequence's score equals its teacher-forced
    log-probability from a plain forward pass of the same model (so the row table handed each beam its own
    history); scores are sorted; beam 1 through the search is the greedy loop up to near-ties in bf16 (the two
    run different kernels: the search's step is not the fused decode block), so its score matches greedy's;
    and the best of four beams scores at least that."""
    say("generate with beams, bf16 consistency")
    from olmo_amd import ops

    for kind in ("olmo2", "olmo2-gqa"):
        cfg = small_cfg(kind)
        cfg.eos_token_id = 3
        model, _ = build_pair(cfg, torch.bfloat16, dev, seed=9)
        ids = torch.randint(4, cfg.vocab_size, (2, 140), generator=torch.Generator().manual_seed(4)).to(dev)

        def teacher_forced(b, toks):
            logits = model(torch.cat([ids[b], toks]).unsqueeze(0)).logits[0]
            lp = ops.log_softmax(logits[ids.shape[1] - 1: -1].contiguous())
            is_end = (toks == cfg.eos_token_id).long()
            after_end = torch.cumsum(is_end, 0) - is_end > 0
            return torch.where(after_end, torch.zeros_like(lp[:, 0]), lp.gather(1, toks.unsqueeze(1)).squeeze(1)).sum().item()

        greedy = model.generate(ids, max_steps=6)
        one = model._generate_beam(ids, None, 6, 1, None, None, None, None, None)
        assert one.token_ids.shape[:2] == (2, 1)
        assert torch.equal(one.token_ids[:, :, :2], greedy.token_ids[:, :, :2])
        assert (one.scores - greedy.scores).abs().max().item() < 0.3
        out = model.generate(ids, max_steps=6, beam_size=4)
        B, K, T = out.token_ids.shape
        assert (B, K) == (2, 4) and bool((out.scores[:, :-1] >= out.scores[:, 1:]).all())
        assert bool((out.scores[:, 0] >= one.scores[:, 0] - 1e-3).all())
        from olmo_amd.beam_search import TopKSampler

        drawn = model.generate(ids, max_steps=5, beam_size=3, sampler=TopKSampler(k=20, temperature=1.3, seed=3))
        assert drawn.token_ids.shape[:2] == (2, 3)
        for b in range(B):  # sampled candidates, true log-probabilities
            for j in range(3):
                assert abs(teacher_forced(b, drawn.token_ids[b, j]) - drawn.scores[b, j].item()) < 0.05 * T
        from olmo_amd.hf import OLMoConfig, OLMoForCausalLM

        hf = OLMoForCausalLM(OLMoConfig.from_model_config(cfg), model=model)
        assert torch.equal(hf.generate(ids, max_new_tokens=6, num_beams=4, loop="captured"), torch.cat([ids, out.token_ids[:, 0]], dim=1))
        for b in range(B):
            assert abs(teacher_forced(b, one.token_ids[b, 0]) - one.scores[b, 0].item()) < 0.05 * T
            for j in range(K):
                tf = teacher_forced(b, out.token_ids[b, j])
                assert abs(tf - out.scores[b, j].item()) < 0.05 * T, (kind, b, j, tf, out.scores[b, j].item())
