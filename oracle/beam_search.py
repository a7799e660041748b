"""TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's beam search
(``olmo/beam_search.py:649-1078``) with the deterministic sampler (``:102-113``), the two final-sequence
scorers (``:449-491``) and the repeated-n-gram constraint (``:593-646``).

Nothing in the product (``olmo_amd/``) may import this module.

``beam_search(step, start_predictions, state, ...)`` follows ``BeamSearch._search`` line by line on CPU
tensors: first step from ``[batch]`` to ``[batch, beam]`` (``:837-912``), then per step the per-node top-k
(``:960-963``), the running sums (``:965-990``), the beam-level top-k (``:992-1012``), backpointers
(``:1019-1020``) and the gather of every state tensor along the group axis (``:1062-1078``) -- the cache
gather the device build replaces by a row table -- and finally the reconstruction from the backpointers
(``:721-747``), the scorer and the sort (``:1030-1045``).

One choice the reference leaves open: ``torch.topk`` does not define the order of equal values.  Here (and on
the device) equal values are taken in ascending index order (a stable descending sort).

Pinned by ``tests/test_oracle_beam_search.py`` against every known-answer case of the reference's own
``tests/beam_search_test.py`` (transition matrices and expected sequences / scores, kept as data in
``tests/golden/beam_search_kat.json``): plain search, batch of one, greedy, single step, early stopping,
short sequences, ``min_steps``, ``per_node_beam_size``, length normalisation with three penalties, and the
n-gram blocking cases (uni-, bi-, trigrams, repeated end tokens) -- and by a brute-force enumeration of all
sequences on a small random chain (with a full-width beam the search is exhaustive).
"""

from __future__ import annotations

import copy
from typing import Callable, Dict, List, Optional, Tuple

import torch

__all__ = ["beam_search", "topk_stable", "length_normalized_score", "NGramBlocker"]


def topk_stable(x: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    v, i = torch.sort(x, dim=-1, descending=True, stable=True)
    return v[..., :k].contiguous(), i[..., :k].contiguous()


def length_normalized_score(predictions: torch.Tensor, log_probs: torch.Tensor, end_index: int,
                            length_penalty: float) -> torch.Tensor:
    """``olmo/beam_search.py:478-491``: tokens before the end token, plus one when the sequence ended."""
    lengths = (predictions != end_index).long().sum(dim=2) + (predictions[:, :, -1] == end_index).long()
    return log_probs / (lengths**length_penalty)


class NGramBlocker:
    """``RepeatedNGramBlockingConstraint`` (``olmo/beam_search.py:593-646``): per (batch, beam) the map
    (n-1)-gram -> tokens that followed it, and the current (n-1)-gram."""

    def __init__(self, ngram_size: int):
        self.n = ngram_size

    def init_state(self, batch: int):
        return [[{"seen": {}, "prefix": []}] for _ in range(batch)]

    def apply(self, state, log_probs: torch.Tensor) -> torch.Tensor:  # [batch, beam, classes], in place
        for i, row in enumerate(state):
            for j, s in enumerate(row):
                banned = s["seen"].get(tuple(s["prefix"]))
                if banned:
                    log_probs[i, j, banned] = torch.finfo(log_probs.dtype).min
        return log_probs

    def update(self, state, prediction: torch.Tensor, backpointer: Optional[torch.Tensor]):
        batch, beam = prediction.shape
        new = [[copy.deepcopy(state[i][0 if backpointer is None else int(backpointer[i, j])]) for j in range(beam)]
               for i in range(batch)]
        for i in range(batch):
            for j in range(beam):
                s, tok = new[i][j], int(prediction[i, j])
                if len(s["prefix"]) == self.n - 1:
                    s["seen"].setdefault(tuple(s["prefix"]), []).append(tok)
                s["prefix"].append(tok)
                if len(s["prefix"]) == self.n:
                    s["prefix"].pop(0)
        return new


def beam_search(step: Callable, start_predictions: torch.Tensor, state: Dict[str, torch.Tensor], end_index: int,
                max_steps: int = 50, beam_size: int = 10, per_node_beam_size: Optional[int] = None,
                min_steps: int = 0, length_penalty: Optional[float] = None, ngram_size: Optional[int] = None,
                ) -> Tuple[torch.Tensor, torch.Tensor]:
    """``step(last_predictions [group], state, timestep) -> (log_probs [group, classes], state)``.  Returns
    ``(predictions [batch, beam, steps], scores [batch, beam])`` sorted by score."""
    B, K = start_predictions.shape[0], beam_size
    PN = per_node_beam_size or beam_size
    blocker = NGramBlocker(ngram_size) if ngram_size else None
    bstate = blocker.init_state(B) if blocker else None
    predictions: List[torch.Tensor] = []
    backpointers: List[torch.Tensor] = []

    lp, state = step(start_predictions, state, 0)
    lp = lp.clone()
    V = lp.shape[1]
    if PN > V:
        raise ValueError("per_node_beam_size exceeds the number of classes")
    fmin = torch.finfo(lp.dtype).min
    if blocker:
        lp = blocker.apply(bstate, lp.unsqueeze(1)).squeeze(1)
    if min_steps >= 1:
        lp[:, end_index] = fmin
    last_lp, cls = topk_stable(lp, K)
    if K == 1 and bool((cls == end_index).all()):
        return cls.unsqueeze(-1), last_lp
    predictions.append(cls)
    after_end = torch.full((B * K, V), fmin, dtype=lp.dtype)
    after_end[:, end_index] = 0.0
    for key, v in state.items():  # every beam starts as a copy of its sequence
        state[key] = v.unsqueeze(1).expand(B, K, *v.shape[1:]).reshape(B * K, *v.shape[1:])
    if blocker:
        bstate = blocker.update(bstate, cls, None)

    for t in range(max_steps - 1):
        last = predictions[-1].reshape(B * K)
        if bool((last == end_index).all()):
            break
        lp, state = step(last, state, t + 1)
        lp = lp.clone()
        if blocker:
            lp = blocker.apply(bstate, lp.view(B, K, -1)).view(B * K, -1)
        if t + 2 <= min_steps:
            lp[:, end_index] = fmin
        lp = torch.where((last == end_index).unsqueeze(1), after_end, lp)  # a finished beam can only repeat the end
        node_lp, node_cls = topk_stable(lp, PN)
        summed = (node_lp.view(B, K, PN) + last_lp.unsqueeze(2)).reshape(B, K * PN)
        last_lp, pick = topk_stable(summed, K)
        predictions.append(node_cls.reshape(B, K * PN).gather(1, pick))
        bp = torch.div(pick, PN, rounding_mode="trunc")
        backpointers.append(bp)
        rows = (bp + torch.arange(B).unsqueeze(1) * K).reshape(-1)
        for key, v in state.items():
            state[key] = v.index_select(0, rows)
        if blocker:
            bstate = blocker.update(bstate, predictions[-1], bp)

    seq = [predictions[-1]]
    if backpointers:
        cur = backpointers[-1]
        for t in range(len(predictions) - 2, 0, -1):
            seq.append(predictions[t].gather(1, cur))
            cur = backpointers[t - 1].gather(1, cur)
        seq.append(predictions[0].gather(1, cur))
    allp = torch.stack(list(reversed(seq)), dim=2)
    final = last_lp if length_penalty is None else length_normalized_score(allp, last_lp, end_index, length_penalty)
    scores, order = torch.sort(final, dim=1, descending=True, stable=True)
    return allp.gather(1, order.unsqueeze(-1).expand_as(allp)), scores
