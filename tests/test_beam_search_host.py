"""Host-side pieces of ``olmo_amd.beam_search`` and of the oracle's search that need no GPU: the n-gram constraint's
state (the reference's own cases, ``tests/beam_search_test.py:519-592``), the scorers, constructor checks."""

import pytest
import torch

from olmo_amd.beam_search import (BeamSearch, LengthNormalizedSequenceLogProbabilityScorer,
                                  RepeatedNGramBlockingConstraint, SequenceLogProbabilityScorer, TopKSampler, TopPSampler)
from oracle.beam_search import NGramBlocker, length_normalized_score


def _state():
    return [
        [{"current_prefix": [0, 1], "seen_ngrams": {}}, {"current_prefix": [2, 3], "seen_ngrams": {(2, 3): [4]}}],
        [{"current_prefix": [4, 5], "seen_ngrams": {(8, 9): []}}, {"current_prefix": [6, 7], "seen_ngrams": {(6, 7): [0, 1, 2]}}],
    ]


def test_ngram_constraint_init_apply_update():
    c = RepeatedNGramBlockingConstraint(3)
    st = c.init_state(2)
    assert len(st) == 2 and all(len(b) == 1 and b[0] == {"seen_ngrams": {}, "current_prefix": []} for b in st)
    lp = torch.rand(2, 2, 10)
    c.apply(_state(), lp)
    banned = torch.nonzero(lp == torch.finfo(lp.dtype).min).tolist()
    assert sorted(banned) == [[0, 1, 4], [1, 1, 0], [1, 1, 1], [1, 1, 2]]
    new = c.update_state(_state(), torch.tensor([[5, 6], [0, 3]]), torch.tensor([[1, 1], [0, 1]]))
    assert new == [
        [{"current_prefix": [3, 5], "seen_ngrams": {(2, 3): [4, 5]}}, {"current_prefix": [3, 6], "seen_ngrams": {(2, 3): [4, 6]}}],
        [{"current_prefix": [5, 0], "seen_ngrams": {(8, 9): [], (4, 5): [0]}},
         {"current_prefix": [7, 3], "seen_ngrams": {(6, 7): [0, 1, 2, 3]}}],
    ]


def test_oracle_blocker_agrees_with_the_reference_cases():
    """The oracle keeps the same books under other key names."""
    b = NGramBlocker(3)
    st = [[{"prefix": s["current_prefix"], "seen": s["seen_ngrams"]} for s in row] for row in _state()]
    lp = torch.rand(2, 2, 10)
    b.apply(st, lp)
    assert sorted(torch.nonzero(lp == torch.finfo(lp.dtype).min).tolist()) == [[0, 1, 4], [1, 1, 0], [1, 1, 1], [1, 1, 2]]
    new = b.update(st, torch.tensor([[5, 6], [0, 3]]), torch.tensor([[1, 1], [0, 1]]))
    assert new[0][0] == {"prefix": [3, 5], "seen": {(2, 3): [4, 5]}} and new[1][1] == {"prefix": [7, 3], "seen": {(6, 7): [0, 1, 2, 3]}}
    assert new[1][0] == {"prefix": [5, 0], "seen": {(8, 9): [], (4, 5): [0]}}


def test_scorers():
    preds = torch.tensor([[[1, 2, 5, 5], [1, 2, 3, 4]]])
    lp = torch.tensor([[-1.0, -2.0]])
    assert torch.equal(SequenceLogProbabilityScorer().score(preds, lp, 5), lp)
    # first beam: 2 tokens + the end token; second: 4 tokens, never ended
    got = LengthNormalizedSequenceLogProbabilityScorer(length_penalty=2.0).score(preds, lp, 5)
    assert torch.allclose(got, torch.tensor([[-1.0 / 9, -2.0 / 16]]))
    assert torch.allclose(length_normalized_score(preds, lp, 5, 2.0), got)


def test_constructor_checks():
    for bad in (dict(max_steps=0), dict(beam_size=0), dict(per_node_beam_size=0), dict(min_steps=-1),
                dict(min_steps=11, max_steps=10)):
        with pytest.raises(ValueError):
            BeamSearch(5, **bad)
    bs = BeamSearch(5, beam_size=4)
    assert bs.per_node_beam_size == 4 and bs.min_steps == 0 and bs.max_steps == 50 and bs.sampler.greedy
    with pytest.raises(ValueError):
        TopPSampler(p=-0.1)
    with pytest.raises(ValueError):
        TopKSampler(k=0).check(10)
    with pytest.raises(RuntimeError):  # the search itself runs on the device only
        bs.search(torch.zeros(2, dtype=torch.long), {}, lambda last, st: (torch.zeros(2, 6), st))
