"""Greedy decoding over the KV cache: prefill once, then one token per step.

Stands in for the two drivers the reference reaches ``OLMo.forward`` through: the HF
``generate`` loop behind ``hf_olmo/modeling_olmo.py:150-160`` and ``OLMo.generate`` with beam 1
(``olmo/model.py:1603-1728``; the deterministic sampler takes ``topk(1)`` of the log-softmax,
``olmo/beam_search.py:102-113``, i.e. the arg-max of the logits).

The decode step (embedding, all blocks, final norm, head, arg-max, position increment) is
launch-bound in Python, so it is captured once into a HIP graph and replayed: every kernel reads
the current position from device memory, the new token is written where the next step's
embedding lookup reads it, and no launch argument changes between steps.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import ops

__all__ = ["greedy_generate", "DecodeSession"]  # greedy_generate also samples (its ``sampling`` argument)


class DecodeSession:
    """State of one batched decode after its prefill: greedy, or sampled when ``sampling`` holds
    ``temperature`` / ``top_k`` / ``top_p`` / ``seed`` (the draw then runs on the device inside the step, with
    the device-side position as the random-number counter, so a captured step draws afresh on every replay)."""

    def __init__(self, model, cache, first_ids: torch.Tensor, key_bias_full: Optional[torch.Tensor],
                 sampling: Optional[dict] = None):
        self.model = model
        self.sampling = sampling
        self.logprob = torch.zeros(first_ids.shape[0], dtype=torch.float32, device=first_ids.device)
        self.cache = cache
        self.B = first_ids.shape[0]
        self.ids = first_ids.view(self.B, 1).contiguous()  # token to feed next; rewritten by every step
        self.key_bias = key_bias_full
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.logits: Optional[torch.Tensor] = None
        # rotary rows of the position about to be written, refreshed on the device after every step
        sin, cos = model._rope
        cache.rope_now = torch.empty(2 * sin.shape[1], dtype=torch.float32, device=sin.device)
        ops.rope_advance(cache.length_dev, 0, sin, cos, cache.rope_now)
        # greedy: the step's last launch picks the token, looks up its embedding row for the next step and advances
        # the position (three launches otherwise, and the next step's first)
        wte = model.transformer["wte"].weight.data
        self.x_next = model.transformer["wte"](self.ids) if sampling is None and wte.is_contiguous() else None

    def _step_kernels(self) -> None:
        m = self.model
        x = self.x_next if self.x_next is not None else m.transformer["wte"](self.ids)
        logits, _ = m._forward_tokens(x, self.cache, self.B, 1, 0, self.key_bias, self.cache.length_dev, False)
        self.logits = logits
        if self.x_next is not None:
            ops.greedy_next(logits.view(self.B, -1), self.ids.view(self.B), m.transformer["wte"].weight.data, self.x_next,
                            self.cache.length_dev, *m._rope, self.cache.rope_now)
            return
        if self.sampling is None:
            ops.argmax(logits.view(self.B, -1), out=self.ids.view(self.B))
        else:
            ops.sample(logits.view(self.B, -1), counter_dev=self.cache.length_dev, out=self.ids.view(self.B),
                       logprob=self.logprob, **self.sampling)
        ops.rope_advance(self.cache.length_dev, 1, *m._rope, self.cache.rope_now)

    def feed(self, ids: torch.Tensor) -> None:
        """Replace the token that the next step reads (``self.ids`` is what the last step chose): writes it where
        the step looks for it, the embedding row included when the greedy step keeps that ahead."""
        self.ids.copy_(ids.view(self.B, 1))
        if self.x_next is not None:
            self.x_next.copy_(self.model.transformer["wte"](self.ids))

    def step(self) -> None:
        """Advance by one token: afterwards ``self.ids`` holds the new token of every sequence.  (A greedy step has
        already looked up that token's embedding row for the step after it: to feed another token use :meth:`feed`.)"""
        if self.cache.length + 1 > self.cache.capacity:
            raise ValueError("KV cache capacity exceeded")
        if self.graph is not None:
            self.graph.replay()
        else:
            self._step_kernels()
        self.cache.length += 1  # host mirror of the device counter

    def capture(self) -> None:
        """Record one decode step into a HIP graph (call after at least one eager ``step`` so that
        the attention workspace already exists)."""
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self._step_kernels()
        self.graph = g


def _prefill(model, input_ids, attention_mask, sampling: Optional[dict] = None,
             attention_bias: Optional[torch.Tensor] = None, key_bias_extra: Optional[torch.Tensor] = None):
    """``key_bias_extra``: ``attention_bias`` as a per-key bias over prompt + new tokens (see
    ``OLMo.key_bias_from_attention_bias``), for the decode steps that follow."""
    out = model(input_ids, attention_mask=attention_mask, attention_bias=attention_bias, use_cache=True,
                last_logits_only=True)
    cache = out.attn_key_values[0].cache
    B = input_ids.shape[0]
    if sampling is None:
        first = ops.argmax(out.logits.view(B, -1))
    else:  # counter: the position of the token being drawn, as in the decode steps
        first, _ = ops.sample(out.logits.view(B, -1), counter=input_ids.shape[1], **sampling)
    key_bias_full = None
    if attention_mask is not None:
        am = attention_mask.to(model.device, torch.float32).view(B, -1)
        key_bias_full = torch.zeros(B, cache.capacity, dtype=torch.float32, device=model.device)
        key_bias_full[:, : am.shape[1]] = (1.0 - am) * torch.finfo(torch.float32).min
    if key_bias_extra is not None:
        if key_bias_full is None:
            key_bias_full = torch.zeros(B, cache.capacity, dtype=torch.float32, device=model.device)
        key_bias_full[:, : key_bias_extra.shape[1]] += key_bias_extra
    return out, cache, first, key_bias_full


@torch.no_grad()
def greedy_generate(model, input_ids: torch.Tensor, attention_mask: Optional[torch.Tensor], max_new_tokens: int,
                    use_graph: bool = True, eos_token_id: Optional[int] = None, pad_token_id: Optional[int] = None,
                    return_scores: bool = False, return_logits: bool = False, sampling: Optional[dict] = None,
                    stop_when_all_ended: bool = False, attention_bias: Optional[torch.Tensor] = None):
    """Returns ``tokens [B, max_new_tokens]`` (and, on request, the summed log-probabilities of the
    chosen tokens and / or the per-step logits).  Runs ``max_new_tokens`` steps; with
    ``eos_token_id`` the tokens after a sequence's first EOS are replaced by ``pad_token_id`` and add nothing to
    the score, and with ``stop_when_all_ended`` the loop also ends (and the result is cut) once every sequence has
    emitted it, as the reference's search does.
    ``sampling`` (``temperature``, ``top_k``, ``top_p``, ``seed``) draws the tokens instead of taking the
    arg-max; the same seed and prompt give the same tokens."""
    if max_new_tokens < 1:
        raise ValueError("max_new_tokens must be >= 1")
    input_ids = input_ids.to(model.device)
    B, T0 = input_ids.shape
    if T0 + max_new_tokens - 1 > model.max_cache_len:
        raise ValueError(f"prompt {T0} + {max_new_tokens} new tokens exceeds max_cache_len {model.max_cache_len}")
    key_bias_extra = None
    if attention_bias is not None:  # olmo/model.py:1607,1645-1651: one bias over prompt + generated tokens
        key_bias_extra = model.key_bias_from_attention_bias(attention_bias, B, 0, T0 + max_new_tokens - 1)
    out, cache, first, key_bias_full = _prefill(model, input_ids, attention_mask, sampling, attention_bias, key_bias_extra)
    sess = DecodeSession(model, cache, first, key_bias_full, sampling)
    tokens = torch.empty(B, max_new_tokens, dtype=torch.int64, device=model.device)
    tokens[:, 0] = sess.ids.view(B)
    all_logits = [out.logits[:, -1].clone()] if return_logits else None
    # scores: the chosen token's log-probability per step.  The logits of a step are kept only until a batch of
    # steps has been turned into those numbers (a [B, 64, V] block at a time, not steps x V for the whole run)
    tok_lp = torch.zeros(B, max_new_tokens, dtype=torch.float32, device=model.device) if return_scores else None
    pending = [(0, out.logits[:, -1].clone())] if return_scores else []

    def settle():
        if not pending:
            return
        idx = torch.tensor([i for i, _ in pending], device=model.device)
        lp = torch.log_softmax(torch.stack([l for _, l in pending], dim=1).float(), dim=-1)
        tok_lp[:, idx] = lp.gather(-1, tokens[:, idx].unsqueeze(-1)).squeeze(-1)
        pending.clear()

    steps = max_new_tokens
    for i in range(1, max_new_tokens):
        if stop_when_all_ended and eos_token_id is not None and i % 16 == 0:
            # the search ends once every sequence has emitted the end token (olmo/beam_search.py:918-923); looked at
            # every 16 steps only: the check is a host synchronisation
            if bool((tokens[:, :i] == eos_token_id).any(dim=1).all()):
                steps = i
                break
        if use_graph and sess.graph is None and i == 3:
            sess.capture()
        sess.step()
        tokens[:, i] = sess.ids.view(B)
        if all_logits is not None:
            all_logits.append(sess.logits.view(B, -1).clone())
        if return_scores:
            pending.append((i, sess.logits.view(B, -1).clone()))
            if len(pending) >= 64:
                settle()
    settle()
    model.relay_check()
    ops.streamk_check()  # a prefill GEMM that gave a tile up as NaN is an error here, not a silent bad token
    tokens = tokens[:, :steps]
    result = [tokens]
    after = None
    if eos_token_id is not None:
        pad = eos_token_id if pad_token_id is None else pad_token_id
        seen = (tokens == eos_token_id).cumsum(dim=1)
        after = (seen - (tokens == eos_token_id).to(seen.dtype)) > 0
        tokens = torch.where(after, torch.full_like(tokens, pad), tokens)
        if stop_when_all_ended:  # as long as the longest sequence, its end token included
            keep = int((~after).sum(dim=1).max().item())
            tokens, after = tokens[:, :keep], after[:, :keep]
        result[0] = tokens
    if return_scores:
        # log-probability bookkeeping of the search (olmo/model.py:1705, beam_search.py:1003-1019);
        # not on the timed path, so plain torch on the saved logits.  An ended sequence adds nothing
        # (beam_search.py:948-957: the forced end token has log-probability 0).
        tok_lp = tok_lp[:, : tokens.shape[1]]  # of the tokens as generated (the padding written over them adds nothing)
        if after is not None:
            tok_lp = tok_lp.masked_fill(after, 0.0)
        result.append(tok_lp.sum(dim=1))
    if return_logits:
        result.append(torch.stack(all_logits[: tokens.shape[1]], dim=1))
    return result[0] if len(result) == 1 else tuple(result)
