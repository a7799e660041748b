"""Pins ``oracle/beam_search.py`` (CPU): every known-answer case the reference's own
``tests/beam_search_test.py`` holds (kept as data in ``tests/golden/beam_search_kat.json``), and an exhaustive
enumeration on a small random chain."""

import itertools
import json
import math
import os

import numpy as np
import pytest
import torch

from oracle.beam_search import beam_search

KAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "beam_search_kat.json")))


def chain_step(matrix: torch.Tensor):
    def step(last, state, timestep):
        return torch.log(matrix[last]), state
    return step


@pytest.mark.parametrize("case", KAT["cases"], ids=[c["name"] for c in KAT["cases"]])
def test_reference_known_answers(case):
    m = torch.tensor(KAT["matrices"][case["matrix"]])
    top, scores = beam_search(chain_step(m), torch.full((case["batch_size"],), KAT["start_token"]), {},
                              KAT["end_index"], max_steps=case["max_steps"], beam_size=case["beam_size"],
                              per_node_beam_size=case.get("per_node_beam_size"), min_steps=case.get("min_steps", 0),
                              length_penalty=case.get("length_penalty"), ngram_size=case.get("ngram_size"))
    assert list(top.shape[:2]) == [case["batch_size"], case["beam_size"]]
    np.testing.assert_array_equal(top[0].numpy(), np.array(case["expected_top_k"]))
    expected = np.log(np.array(case["expected_probs"]))
    if "length_norm" in case:
        expected = expected / np.array(case["length_norm"])
    np.testing.assert_allclose(scores[0].numpy(), expected, rtol=KAT["rtol"])


def test_state_follows_backpointers():
    """``tests/beam_search_test.py:149-180``: a state tensor ends up repeated per beam (all beams of this chain
    descend from their own sequence)."""
    m = torch.tensor(KAT["matrices"]["T"])
    foo = torch.tensor([[1, 0, 1], [2, 0, 1], [0, 0, 1], [1, 1, 1], [0, 0, 0]])
    seen = {}

    def step(last, state, timestep):
        seen["foo"] = state["foo"]
        return torch.log(m[last]), state

    beam_search(step, torch.zeros(5, dtype=torch.long), {"foo": foo}, 5, max_steps=10, beam_size=3)
    np.testing.assert_array_equal(seen["foo"].numpy(), foo.repeat_interleave(3, dim=0).numpy())


def test_full_width_beam_is_exhaustive():
    """Two steps with beam = per-node width = number of classes: the first step keeps every class, so the
    second step's cut must be the brute-force top of all two-token sequences (end token absorbing at no
    cost)."""
    g = torch.Generator().manual_seed(3)
    V, steps, end = 6, 2, 5
    m = torch.rand(V, V, generator=g).double()
    m = m / m.sum(dim=1, keepdim=True)
    top, scores = beam_search(chain_step(m), torch.zeros(1, dtype=torch.long), {}, end, max_steps=steps,
                              beam_size=V, per_node_beam_size=V)
    best = {}
    for seq in itertools.product(range(V), repeat=steps):
        lp, last, ended = 0.0, 0, False
        for tok in seq:
            if ended:
                lp += 0.0 if tok == end else -math.inf
            else:
                lp += math.log(m[last, tok])
            ended = ended or tok == end
            last = tok
        if lp > -math.inf:
            best[seq] = lp
    ranked = sorted(best.items(), key=lambda kv: -kv[1])[: top.shape[1]]
    got = {tuple(int(t) for t in top[0, j]): float(scores[0, j]) for j in range(top.shape[1])}
    for seq, lp in ranked:
        assert seq in got and abs(got[seq] - lp) < 1e-9
