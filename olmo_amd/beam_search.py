"""The samplers of ``olmo/beam_search.py`` for beam size 1, as parameter holders for the device-side
sampling step (``olmo355_sample``): same class names, constructor arguments, defaults and argument checks.

``OLMo.generate(..., sampler=TopPSampler(p=0.9))`` then draws one token per step on the GPU inside the
captured decode step.  Beam widths above 1, ``GumbelSampler``, constraints and final-sequence scorers
(``olmo/beam_search.py:280-1078``) are not implemented.
"""

from __future__ import annotations

__all__ = ["Sampler", "DeterministicSampler", "MultinomialSampler", "TopKSampler", "TopPSampler"]


class Sampler:
    """Base class (``olmo/beam_search.py:72-99``); ``params()`` is what the device kernel takes."""

    temperature: float = 1.0
    top_k: int = 0
    top_p: float = 1.0
    greedy: bool = False

    def params(self) -> dict:
        return {"temperature": float(self.temperature or 1.0), "top_k": int(self.top_k), "top_p": float(self.top_p)}


class DeterministicSampler(Sampler):
    """``topk(log_probs, 1)``: the arg-max (``olmo/beam_search.py:102-114``)."""

    greedy = True


class MultinomialSampler(Sampler):
    """``olmo/beam_search.py:117-146``."""

    def __init__(self, temperature: float = 1.0, with_replacement: bool = False) -> None:
        self.temperature = temperature
        self.with_replacement = with_replacement


class TopKSampler(Sampler):
    """``olmo/beam_search.py:149-196``."""

    def __init__(self, k: int = 1, temperature: float = 1.0, with_replacement: bool = False):
        self.k = k
        self.top_k = k
        self.temperature = temperature or 1.0
        self.with_replacement = with_replacement

    def check(self, vocab: int) -> None:
        if not 1 <= self.k <= vocab:
            raise ValueError(
                "k must be a postive integer no less than per_node_beam_size and no greater than vocabulary size"
            )  # the reference's message, :178-181


class TopPSampler(Sampler):
    """``olmo/beam_search.py:199-277``."""

    def __init__(self, p: float = 0.9, temperature: float = 1.0, with_replacement: bool = False):
        if p < 0.0 or p > 1.0:
            raise ValueError("p must be a positive float no greater than 1.0")  # :227-228
        self.p = p
        self.top_p = p
        self.temperature = temperature or 1.0
        self.with_replacement = with_replacement
