"""``olmo/beam_search.py`` on the device: the samplers, the final-sequence scorers, the constraints and
``BeamSearch`` itself, same class names, constructor arguments, defaults and argument checks.

Beam size 1: the samplers are parameter holders for the device-side sampling step (``olmo355_sample``);
``OLMo.generate(..., sampler=TopPSampler(p=0.9))`` draws one token per step on the GPU inside the captured
decode step.  Beam sizes above 1: ``BeamSearch`` below; the samplers' ``sample_nodes`` draw per-node candidates
on the device (Gumbel-perturbed log-weights + top-k), as does the ``GumbelSampler``'s stochastic beam search.
"""

from __future__ import annotations

import copy
import warnings
from inspect import signature
from typing import Callable, List, Optional

import torch

__all__ = ["Sampler", "DeterministicSampler", "MultinomialSampler", "TopKSampler", "TopPSampler", "GumbelSampler",
           "FinalSequenceScorer", "SequenceLogProbabilityScorer", "LengthNormalizedSequenceLogProbabilityScorer",
           "Constraint", "RepeatedNGramBlockingConstraint", "BeamSearch"]


class Sampler:
    """Base class (``olmo/beam_search.py:44-99``).  Two uses: ``params()`` is what the device-side sampling step of
    a beam-1 generation takes; ``sample_nodes`` / ``sample_beams`` are what :class:`BeamSearch` calls, on float32
    device tensors ``[rows, examples]``, returning ``(log_probs, indices, state)`` like the reference.  Draws are
    made by perturbing log-weights with Gumbel noise and taking the top k (k draws without replacement from the
    softmax; the reference calls ``torch.multinomial``), with noise from ``(seed, draw number)``: a sampler
    object reproduces its draws after ``init_state``; the reference's random stream is not reproduced."""

    temperature: float = 1.0
    top_k: int = 0
    top_p: float = 1.0
    greedy: bool = False
    with_replacement: bool = False
    seed: int = 0
    _draws: int = 0

    def params(self) -> dict:
        return {"temperature": float(self.temperature or 1.0), "top_k": int(self.top_k), "top_p": float(self.top_p)}

    def init_state(self, start_class_log_probabilities: torch.Tensor, batch_size: int, num_classes: int) -> dict:
        self._draws = 0
        return {}

    def sample_nodes(self, log_probs: torch.Tensor, per_node_beam_size: int, state: dict):
        raise NotImplementedError

    def sample_beams(self, log_probs: torch.Tensor, beam_size: int, state: dict):
        """The ``beam_size`` best, deterministically (``olmo/beam_search.py:94-99``)."""
        from . import ops

        v, i = ops.topk(log_probs, beam_size)
        return v, i, {}

    def _draw(self, log_weights: torch.Tensor, k: int, inv_temp: float = 1.0) -> torch.Tensor:
        """Indices ``[rows, k]`` drawn from ``softmax(log_weights * inv_temp)``: without replacement the k largest
        of one perturbed copy, with replacement the largest of k independent ones."""
        from . import ops

        self._draws += 1
        if not self.with_replacement:
            return ops.topk(ops.gumbel_perturb(log_weights, inv_temp, self.seed, self._draws << 16), k)[1]
        return torch.cat([ops.topk(ops.gumbel_perturb(log_weights, inv_temp, self.seed, (self._draws << 16) + j + 1), 1)[1]
                          for j in range(k)], dim=-1)


class DeterministicSampler(Sampler):
    """``topk(log_probs, k)`` (``olmo/beam_search.py:102-114``)."""

    greedy = True

    def sample_nodes(self, log_probs, per_node_beam_size, state):
        from . import ops

        v, i = ops.topk(log_probs, per_node_beam_size)
        return v, i, state


class MultinomialSampler(Sampler):
    """``olmo/beam_search.py:117-146``."""

    def __init__(self, temperature: float = 1.0, with_replacement: bool = False, seed: int = 0) -> None:
        self.temperature = temperature
        self.with_replacement = with_replacement
        self.seed = seed

    def sample_nodes(self, log_probs, per_node_beam_size, state):
        idx = self._draw(log_probs, per_node_beam_size, 1.0 / float(self.temperature or 1.0))
        return log_probs.gather(1, idx), idx, state


class TopKSampler(Sampler):
    """``olmo/beam_search.py:149-203``."""

    def __init__(self, k: int = 1, temperature: float = 1.0, with_replacement: bool = False, seed: int = 0):
        self.k = k
        self.top_k = k
        self.temperature = temperature or 1.0
        self.with_replacement = with_replacement
        self.seed = seed

    def check(self, vocab: int, at_least: int = 1) -> None:
        if not at_least <= self.k <= vocab or self.k < 1:
            raise ValueError(
                "k must be a postive integer no less than per_node_beam_size and no greater than vocabulary size"
            )  # the reference's message, :175-178

    def sample_nodes(self, log_probs, per_node_beam_size, state):
        from . import ops

        self.check(log_probs.size(1), per_node_beam_size)
        top_lp, top_idx = ops.topk(log_probs, self.k)
        idx = top_idx.gather(-1, self._draw(top_lp, per_node_beam_size, 1.0 / float(self.temperature)))
        return log_probs.gather(1, idx), idx, state


class TopPSampler(Sampler):
    """``olmo/beam_search.py:205-289``."""

    def __init__(self, p: float = 0.9, temperature: float = 1.0, with_replacement: bool = False, seed: int = 0):
        if p < 0.0 or p > 1.0:
            raise ValueError("p must be a positive float no greater than 1.0")  # :232-233
        self.p = p
        self.top_p = p
        self.temperature = temperature or 1.0
        self.with_replacement = with_replacement
        self.seed = seed

    def sample_nodes(self, log_probs, per_node_beam_size, state):
        from . import ops

        if not per_node_beam_size <= log_probs.size(1):
            raise ValueError("per_node_beam_size cannot be greater than vocabulary size")
        lp = log_probs if self.temperature == 1.0 else ops.log_softmax(log_probs * (1.0 / float(self.temperature)))
        # the nucleus: sorted descending, everything up to and including the entry at which the cumulative
        # probability reaches p (:252-268); sort and running sum are library calls, the draw is not
        desc, order = torch.sort(lp, dim=-1, descending=True, stable=True)
        reached = torch.cumsum(desc.exp(), dim=-1) >= self.p
        excluded = torch.zeros_like(reached)
        excluded[..., 1:] = reached[..., :-1]
        if not self.with_replacement:
            excluded[..., :per_node_beam_size] = False
        desc = desc.masked_fill(excluded, torch.finfo(torch.float32).min)
        idx = order.gather(-1, self._draw(desc, per_node_beam_size))
        return log_probs.gather(1, idx), idx, state


class GumbelSampler(Sampler):
    """Stochastic beam search (``olmo/beam_search.py:291-421``; Kool, van Hoof, Welling: the Gumbel-top-k trick):
    the ``beam_size`` sequences kept are a sample without replacement from the sequence distribution.  Every
    candidate carries a perturbed log-probability ``G`` drawn conditionally on its parent's (``gumbel_with_max``,
    one device launch per step); beams are cut by ``G``, then ordered by true log-probability."""

    def __init__(self, temperature: float = 1.0, seed: int = 0):
        self.temperature = temperature
        self.seed = seed

    def _gumbel_with_max(self, phi: torch.Tensor, t: torch.Tensor) -> torch.Tensor:
        from . import ops

        self._draws += 1
        return ops.gumbel_with_max(phi, t.reshape(-1).to(torch.float32), self.seed, self._draws)

    def init_state(self, start_class_log_probabilities, batch_size, num_classes):
        self._draws = 0
        zeros = torch.zeros(batch_size, dtype=torch.float32, device=start_class_log_probabilities.device)
        return {"G_phi_S": self._gumbel_with_max(start_class_log_probabilities, zeros)}

    def sample_nodes(self, log_probs, per_node_beam_size, state):
        from . import ops

        lp = log_probs if self.temperature == 1.0 else ops.log_softmax(log_probs * (1.0 / float(self.temperature)))
        phi_new = state["phi_S"].unsqueeze(-1) + lp
        g_new = self._gumbel_with_max(phi_new, state["G_phi_S"])
        top_g, idx = ops.topk(g_new, per_node_beam_size)
        return log_probs.gather(1, idx), idx, {"G_phi_S": top_g}

    def sample_beams(self, log_probs, beam_size, state):
        from . import ops

        batch = log_probs.size(0)
        g, sel = ops.topk(state["G_phi_S"].reshape(log_probs.shape).contiguous(), beam_size)
        sel_lp, order = log_probs.gather(1, sel).sort(dim=-1, descending=True, stable=True)
        sel, g = sel.gather(1, order), g.gather(1, order)
        return sel_lp, sel, {"G_phi_S": g.reshape(batch * beam_size), "phi_S": sel_lp.reshape(batch * beam_size)}


# ---------------------------------------------------------------------------------------------------
# beam search proper (olmo/beam_search.py:424-1078)
# ---------------------------------------------------------------------------------------------------
class FinalSequenceScorer:
    """``olmo/beam_search.py:424-446``."""

    def score(self, predictions: torch.Tensor, log_probabilities: torch.Tensor, end_index: int) -> torch.Tensor:
        raise NotImplementedError


class SequenceLogProbabilityScorer(FinalSequenceScorer):
    """The summed log-probability as it is (``olmo/beam_search.py:449-459``)."""

    def score(self, predictions, log_probabilities, end_index):
        return log_probabilities


class LengthNormalizedSequenceLogProbabilityScorer(FinalSequenceScorer):
    """``log_p / length ** length_penalty``; the length counts the end token when the sequence ended
    (``olmo/beam_search.py:462-491``)."""

    def __init__(self, length_penalty: float = 1.0):
        self.length_penalty = length_penalty

    def score(self, predictions, log_probabilities, end_index):
        lengths = (predictions != end_index).long().sum(dim=2)
        lengths = lengths + (predictions[:, :, -1] == end_index).long()
        return log_probabilities / (lengths**self.length_penalty)


class Constraint:
    """``olmo/beam_search.py:494-590``: per-(batch, beam) host-side state, ``apply`` edits the step's
    log-probabilities ``[batch, beam, classes]`` in place, ``update_state`` follows the backpointers."""

    def init_state(self, batch_size: int):
        raise NotImplementedError

    def apply(self, state, class_log_probabilities: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    @staticmethod
    def _copy_state(state, batch_size: int, beam_size: int, last_backpointer: Optional[torch.Tensor] = None):
        bp = None if last_backpointer is None else last_backpointer.tolist()
        return [[copy.deepcopy(state[i][0 if bp is None else bp[i][j]]) for j in range(beam_size)]
                for i in range(batch_size)]

    def update_state(self, state, last_prediction: torch.Tensor, last_backpointer: Optional[torch.Tensor] = None):
        batch_size, beam_size = last_prediction.size()
        return self._update_state(self._copy_state(state, batch_size, beam_size, last_backpointer), last_prediction)

    def _update_state(self, state, last_prediction: torch.Tensor):
        raise NotImplementedError


class RepeatedNGramBlockingConstraint(Constraint):
    """No n-gram twice in a sequence (``olmo/beam_search.py:593-646``): per beam, the tokens that followed each
    (n-1)-gram so far; the ones that followed the current one are set to the dtype's minimum."""

    def __init__(self, ngram_size: int) -> None:
        self.ngram_size = ngram_size

    def init_state(self, batch_size: int):
        return [[{"seen_ngrams": {}, "current_prefix": []}] for _ in range(batch_size)]

    def apply(self, state, class_log_probabilities: torch.Tensor) -> torch.Tensor:
        rows, cols = [], []
        n_beam = class_log_probabilities.shape[1]
        for i, batch in enumerate(state):
            for j, beam in enumerate(batch):
                banned = beam["seen_ngrams"].get(tuple(beam["current_prefix"]))
                if banned:
                    rows += [i * n_beam + j] * len(banned)
                    cols += banned
        if rows:  # one scatter for the whole step
            flat = class_log_probabilities.view(-1, class_log_probabilities.shape[-1])
            dev = flat.device
            flat[torch.tensor(rows, device=dev), torch.tensor(cols, device=dev)] = torch.finfo(flat.dtype).min
        return class_log_probabilities

    def _update_state(self, state, last_prediction: torch.Tensor):
        preds = last_prediction.tolist()
        for i, batch in enumerate(state):
            for j, beam in enumerate(batch):
                prefix, tok = beam["current_prefix"], preds[i][j]
                if len(prefix) == self.ngram_size - 1:
                    beam["seen_ngrams"].setdefault(tuple(prefix), []).append(tok)
                prefix.append(tok)
                if len(prefix) == self.ngram_size:
                    prefix.pop(0)
        return state


class BeamSearch:
    """``olmo/beam_search.py:649-1078`` with the selections on the device.

    Same constructor, same ``search(start_predictions, start_state, step)`` contract and results: ``step`` returns
    ``(log_probabilities [group, classes], state)``; ``predictions [batch, beam, steps]`` come back sorted by final
    score.  What runs where: the per-node top-k over the classes and the beam-level top-k over
    ``beam * per_node_beam_size`` candidates are ``olmo355_topk`` launches (float32, ties in ascending index
    order); adding the running scores, following backpointers and the final reconstruction touch
    ``[batch, beam]``-sized tensors with torch.  State values are either tensors ``[group, ...]``, gathered along
    the group axis as in the reference (``:1047-1078``), or objects with ``expand_beams(batch, beam)`` and
    ``reorder_beams(backpointer)`` that keep their own books (the KV cache of ``OLMo.generate`` does: it
    updates a table of row numbers instead of moving cache rows)."""

    def __init__(self, end_index: int, *, max_steps: int = 50, beam_size: int = 10,
                 per_node_beam_size: Optional[int] = None, sampler: Optional[Sampler] = None,
                 min_steps: Optional[int] = None, final_sequence_scorer: Optional[FinalSequenceScorer] = None,
                 constraints: Optional[List[Constraint]] = None) -> None:
        if not max_steps > 0:
            raise ValueError("max_steps must be positive")
        if not beam_size > 0:
            raise ValueError("beam_size must be positive")
        if per_node_beam_size is not None and not per_node_beam_size > 0:
            raise ValueError("per_node_beam_size must be positive")
        if min_steps is not None:
            if not min_steps >= 0:
                raise ValueError("min_steps must be non-negative")
            if not min_steps <= max_steps:
                raise ValueError("min_steps must be less than or equal to max_steps")
        self._end_index = end_index
        self.max_steps = max_steps
        self.beam_size = beam_size
        self.per_node_beam_size = per_node_beam_size or beam_size
        self.sampler = sampler or DeterministicSampler()
        self.min_steps = min_steps or 0
        self.final_sequence_scorer = final_sequence_scorer or SequenceLogProbabilityScorer()
        self.constraints = constraints or []

    @staticmethod
    def _reconstruct_sequences(predictions, backpointers):
        """Walk the backpointers from the last step to the first (``olmo/beam_search.py:721-747``); returns
        ``[batch, beam, steps]``."""
        out = [predictions[-1]]
        if backpointers:
            cur = backpointers[-1]
            for t in range(len(predictions) - 2, 0, -1):
                out.append(predictions[t].gather(1, cur))
                cur = backpointers[t - 1].gather(1, cur)
            out.append(predictions[0].gather(1, cur))
        return torch.stack(list(reversed(out)), dim=2)

    def search(self, start_predictions: torch.Tensor, start_state: dict, step: Callable):
        if len(signature(step).parameters) < 3:
            two = step
            step = lambda last, state, timestep: two(last, state)  # noqa: E731
        with torch.no_grad():
            return self._search(start_predictions, start_state, step)

    @staticmethod
    def _f32(log_probs: torch.Tensor) -> torch.Tensor:
        if not log_probs.is_cuda:
            raise RuntimeError("BeamSearch: the step function must return device tensors")
        return log_probs.to(torch.float32).contiguous()

    def _search(self, start_predictions, start_state, step):
        from . import ops

        B, K, PN, end = start_predictions.size(0), self.beam_size, self.per_node_beam_size, self._end_index
        fmin = torch.finfo(torch.float32).min
        predictions: List[torch.Tensor] = []
        backpointers: List[torch.Tensor] = []
        cstates = [c.init_state(B) for c in self.constraints]

        lp, state = step(start_predictions, start_state, 0)
        lp = self._f32(lp)
        V = lp.size(1)
        if PN > V:
            raise ValueError(f"Vocab size ({V:d}) too small relative to per_node_beam_size ({PN:d}).\n"
                             f"Please decrease beam_size or per_node_beam_size.")
        if K > V:
            raise ValueError(f"Vocab size ({V:d}) too small relative to beam_size ({K:d}).")
        sstate = self.sampler.init_state(lp, B, V)  # before the constraints, as in the reference (:851)
        for c, cs in zip(self.constraints, cstates):
            lp = c.apply(cs, lp.unsqueeze(1)).squeeze(1)
        if self.min_steps >= 1:
            lp[:, end] = fmin
        last_lp, cls, sstate = self.sampler.sample_beams(lp, K, sstate)
        if K == 1 and bool((cls == end).all()):
            warnings.warn("Empty sequences predicted. You may want to increase the beam size or ensure "
                          "your step function is working properly.", RuntimeWarning)
            return cls.unsqueeze(-1), last_lp
        predictions.append(cls)

        # what a finished beam proposes: the end token at no cost, anything else at the minimum
        after_end = torch.full((1, V), fmin, dtype=torch.float32, device=lp.device)
        after_end[0, end] = 0.0
        after_v, after_i = ops.topk(after_end, PN)

        self._update_initial_state(state, B)
        for i, c in enumerate(self.constraints):
            cstates[i] = c.update_state(cstates[i], cls)

        for timestep in range(self.max_steps - 1):
            last = predictions[-1].reshape(B * K)
            finished = last == end
            if bool(finished.all()):
                break
            lp, state = step(last, state, timestep + 1)
            lp = self._f32(lp)
            for c, cs in zip(self.constraints, cstates):
                lp = c.apply(cs, lp.view(B, K, -1)).view(B * K, -1)
            if timestep + 2 <= self.min_steps:
                lp[:, end] = fmin
            if getattr(self.sampler, "greedy", False):
                # the top of a finished beam's one-hot row is known: patch the rows instead of building it
                node_lp, node_cls, sstate = self.sampler.sample_nodes(lp, PN, sstate)
                node_lp = torch.where(finished.unsqueeze(1), after_v, node_lp)
                node_cls = torch.where(finished.unsqueeze(1), after_i, node_cls)
            else:  # a sampler may keep state per candidate: give it the rows the reference gives it (:948-957)
                node_lp, node_cls, sstate = self.sampler.sample_nodes(torch.where(finished.unsqueeze(1), after_end, lp),
                                                                      PN, sstate)
            summed = (node_lp.view(B, K, PN) + last_lp.unsqueeze(2)).reshape(B, K * PN)
            last_lp, pick, sstate = self.sampler.sample_beams(summed, K, sstate)
            predictions.append(node_cls.reshape(B, K * PN).gather(1, pick))
            backpointer = torch.div(pick, PN, rounding_mode="trunc")
            backpointers.append(backpointer)
            self._update_state(state, backpointer)
            for i, c in enumerate(self.constraints):
                cstates[i] = c.update_state(cstates[i], predictions[-1], last_backpointer=backpointer)

        if not self.constraints and (not bool(torch.isfinite(last_lp).all()) or bool((last_lp == fmin).any())):
            warnings.warn("Negligible log probabilities encountered ('-inf' or equivalent). "
                          "Some final sequences may not make sense. "
                          "This can happen when the beam size is larger than the number of valid (non-zero "
                          "probability) transitions that the step function produces.", RuntimeWarning)
        all_predictions = self._reconstruct_sequences(predictions, backpointers)
        final = self.final_sequence_scorer.score(all_predictions, last_lp, end)
        scores, order = torch.sort(final, dim=1, descending=True, stable=True)
        return all_predictions.gather(1, order.unsqueeze(-1).expand_as(all_predictions)), scores

    def _update_initial_state(self, state: dict, batch_size: int) -> None:
        """``[batch, ...] -> [batch * beam, ...]``, every beam a copy of its sequence (``:1047-1060``)."""
        for key, v in state.items():
            if v is None:
                continue
            if hasattr(v, "expand_beams"):
                v.expand_beams(batch_size, self.beam_size)
                continue
            rest = v.shape[1:]
            state[key] = v.unsqueeze(1).expand(batch_size, self.beam_size, *rest).reshape(batch_size * self.beam_size, *rest)

    def _update_state(self, state: dict, backpointer: torch.Tensor) -> None:
        """Every beam takes over its parent's state (``:1062-1078``)."""
        B = backpointer.size(0)
        rows = (backpointer + torch.arange(B, device=backpointer.device).unsqueeze(1) * self.beam_size).reshape(-1)
        for key, v in state.items():
            if v is None:
                continue
            if hasattr(v, "reorder_beams"):
                v.reorder_beams(backpointer)
                continue
            state[key] = v.index_select(0, rows.to(v.device))
