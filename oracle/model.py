"""TEST INFRASTRUCTURE ONLY -- pure-torch CPU restatement of the reference's inference
forward pass (``olmo/model.py:1253-1465`` and the functions it reaches).

Nothing in the product (``olmo_amd/``) may import this module; it is the checker used by
``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg.

Covered switches: sequential block, rotary positions, SwiGLU, no biases, no weight tying,
``norm_after`` on or off, RMS (affine) or non-parametric LayerNorm, QK-norm on or off,
dense or int4-group-quantised block Linears, KV cache, ``attention_mask`` padding.

Weights are a flat dict keyed by the reference's state-dict names
(``transformer.wte.weight``, ``transformer.blocks.{i}.att_proj.weight`` ..., for quantised
Linears ``....att_proj.qweight / qzeros / scales``).

Rounding points in a 16-bit activation dtype follow the reference op by op: every Linear
output, residual add, norm (two roundings for RMS), rotary output and SwiGLU product is
rounded to the activation dtype; reductions run in fp32.  Matrix products are evaluated as
fp32 products of the widened operands rounded once, which is what the reference's
``F.linear`` / ``F.scaled_dot_product_attention`` approximate.

Pinned by (tests/test_oracle_model.py): ``F.layer_norm`` for LayerNorm, an fp64 closed form
with explicit rounding for RMSNorm, closed-form and relative-position invariants for RoPE,
``F.scaled_dot_product_attention(is_causal=True)`` and a brute-force softmax for attention,
and the reference's own forward invariants (cache == no cache, padded batch == single:
``tests/model_test.py:188-199``).  No stored golden logits exist in the reference, so the *composition*
(``_block`` / ``_attention`` / ``forward``: norm placement, full-width QK-norm, q | k | v and up | gate split
orders, cache path, padding bias) is pinned by tests/test_oracle_composition.py against logits of
``transformers``' own ``Olmo2ForCausalLM`` (MHA, GQA) and ``OlmoForCausalLM`` (with and without ``clip_qkv``)
on seeded weights mapped the way ``scripts/convert_olmo2_to_hf.py:110-163`` maps them (fixture
tests/golden/hf_olmo2_kat.npz), with negative cases for swapped up / gate, swapped block norms and per-head
QK-norm.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F

from . import w4

__all__ = ["OracleModel", "rms_norm", "layer_norm_np", "rope_tables", "apply_rope", "swiglu", "attention"]


def rms_norm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """``RMSLayerNorm.forward`` (``olmo/model.py:241-255``): fp32 normalise, round to the
    input dtype, *then* multiply by the weight in the input dtype."""
    og = x.dtype
    xf = x.to(torch.float32)
    var = xf.pow(2).mean(-1, keepdim=True)
    y = (xf * torch.rsqrt(var + eps)).to(og)
    if weight is not None:
        return weight.to(og) * y
    return y


def layer_norm_np(x: torch.Tensor, eps: float) -> torch.Tensor:
    """Non-parametric ``LayerNorm.forward`` (``olmo/model.py:212-225``)."""
    return F.layer_norm(x, (x.shape[-1],), None, None, eps)


def rope_tables(head_dim: int, theta: float, seq_len: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """``RotaryEmbedding.get_rotary_embedding`` (``olmo/model.py:285-296``): fp32 ``[L, hd]`` sin, cos."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float) / head_dim))
    seq = torch.arange(seq_len, dtype=torch.float)
    freqs = seq[:, None] * inv_freq[None, :]
    pos = torch.cat((freqs, freqs), dim=-1)
    return pos.sin(), pos.cos()


def apply_rope(t: torch.Tensor, sin: torch.Tensor, cos: torch.Tensor) -> torch.Tensor:
    """``apply_rotary_pos_emb`` + ``rotate_half`` in fp32 (``olmo/model.py:298-324``).
    ``t``: ``[B, H, T, hd]``; ``sin``/``cos``: ``[T, hd]`` rows for the positions of ``t``."""
    tf = t.to(torch.float32)
    hd = tf.shape[-1]
    x1, x2 = tf[..., : hd // 2], tf[..., hd // 2 :]
    rot = torch.cat((-x2, x1), dim=-1)
    return ((tf * cos) + (rot * sin)).to(t.dtype)


def swiglu(x: torch.Tensor) -> torch.Tensor:
    """``SwiGLU.forward`` (``olmo/model.py:365-368``): first half is *up*, second half the gate."""
    up, gate = x.chunk(2, dim=-1)
    return F.silu(gate) * up


def _finfo_min(dtype: torch.dtype) -> float:
    return torch.finfo(dtype).min


def attention(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, bias: Optional[torch.Tensor], act_dtype: torch.dtype
) -> torch.Tensor:
    """``softmax(q k^T / sqrt(hd) + bias) v`` (``olmo/model.py:579-586``) in fp32 on the
    widened operands; ``bias`` None means causal with the queries at the *end* of the keys.
    ``q [B,H,T,hd]``, ``k,v [B,Hkv,L,hd]``; GQA repeats kv heads (``:570-577``)."""
    B, H, T, hd = q.shape
    Hkv, L = k.shape[1], k.shape[2]
    if Hkv != H:
        k = k.repeat_interleave(H // Hkv, dim=1)
        v = v.repeat_interleave(H // Hkv, dim=1)
    s = (q.to(torch.float32) @ k.to(torch.float32).transpose(-1, -2)) / math.sqrt(hd)
    if bias is None:
        i = torch.arange(T)[:, None] + (L - T)
        j = torch.arange(L)[None, :]
        s = s.masked_fill(j > i, float("-inf"))
    else:
        s = s + bias.to(torch.float32)
    p = torch.softmax(s, dim=-1)
    return (p @ v.to(torch.float32)).to(act_dtype)


class OracleModel:
    """Holds a config (any object with the reference's ``ModelConfig`` attribute names) and a
    weight dict; ``forward`` mirrors ``OLMo.forward``'s arguments and returns
    ``(logits, attn_key_values)`` with the cache in the reference's form: per layer ``(k, v)``
    of shape ``[B, n_kv_heads, L, hd]``, ``k`` post-QK-norm and *pre*-RoPE (``olmo/model.py:615-625``)."""

    def __init__(self, cfg, weights: Dict[str, torch.Tensor], act_dtype: torch.dtype, group_size: int = 128,
                 cache_weights: bool = True):
        """``cache_weights=False`` widens / dequantises the weight on every call, as the reference's
        ``QuantLinear.forward`` does (``AGQ:qlinear_cuda_old.py:236-287``); used when timing."""
        self.cfg = cfg
        self.cache_weights = cache_weights
        self.w = weights
        self.act = act_dtype
        self.group_size = group_size
        self._wf32: Dict[str, torch.Tensor] = {}
        self._rope: Optional[Tuple[torch.Tensor, torch.Tensor]] = None

    # -- linear layers ---------------------------------------------------------------------
    def _weight_kn_f32(self, prefix: str) -> torch.Tensor:
        """fp32 ``[K, N]`` operand of Linear ``prefix``, dense or dequantised, cached."""
        if prefix in self._wf32:
            return self._wf32[prefix]
        if prefix + ".weight" in self.w:
            w = self.w[prefix + ".weight"].to(torch.float32).t()
        else:
            w = w4.dequantize(
                self.w[prefix + ".qweight"], self.w[prefix + ".qzeros"], self.w[prefix + ".scales"], self.group_size,
                self.w.get(prefix + ".g_idx"),
            ).to(torch.float32)
        if self.cache_weights:
            self._wf32[prefix] = w = w.contiguous()
        return w

    def linear(self, prefix: str, x: torch.Tensor) -> torch.Tensor:
        """``nn.Linear`` without bias, or ``QuantLinear.forward``'s dequantise-then-matmul
        (``AGQ:qlinear_cuda_old.py:284-290``: the product in the activation dtype, then ``+ bias`` when the
        layer has a bias buffer), result in the activation dtype."""
        y = (x.to(torch.float32) @ self._weight_kn_f32(prefix)).to(self.act)
        b = self.w.get(prefix + ".bias")
        if b is not None and prefix + ".qweight" in self.w:
            y = (y.to(torch.float32) + b.to(torch.float32)).to(self.act)
        return y

    def drop_cache(self):
        self._wf32.clear()

    # -- norms -----------------------------------------------------------------------------
    def _norm(self, name: str, x: torch.Tensor) -> torch.Tensor:
        c = self.cfg
        if c.layer_norm_type == "rms":
            return rms_norm(x, self.w.get(name + ".weight"), c.layer_norm_eps)
        return layer_norm_np(x, c.layer_norm_eps)

    # -- attention block -------------------------------------------------------------------
    def _attention(self, i, q, k, v, bias, layer_past, use_cache):
        c = self.cfg
        B, T, C = q.shape
        hd = c.d_model // c.n_heads
        pre = f"transformer.blocks.{i}."
        if c.attention_layer_norm:  # olmo/model.py:603-605: over the full projected width
            q = rms_norm(q, self.w.get(pre + "q_norm.weight"), c.layer_norm_eps)
            k = rms_norm(k, self.w.get(pre + "k_norm.weight"), c.layer_norm_eps)
        q = q.view(B, T, c.n_heads, hd).transpose(1, 2)
        k = k.view(B, T, c.effective_n_kv_heads, hd).transpose(1, 2)
        v = v.view(B, T, c.effective_n_kv_heads, hd).transpose(1, 2)
        if layer_past is not None:
            k = torch.cat((layer_past[0], k), dim=-2)
            v = torch.cat((layer_past[1], v), dim=-2)
        present = (k, v) if use_cache else None
        L = k.shape[-2]
        if c.rope:
            if self._rope is None or self._rope[0].shape[0] < L:
                self._rope = rope_tables(hd, c.rope_theta, max(L, c.max_sequence_length))
            sin, cos = self._rope[0][:L], self._rope[1][:L]
            q = apply_rope(q, sin[L - T : L], cos[L - T : L])
            k = apply_rope(k, sin, cos)
        if bias is not None:
            # _cast_attn_bias (olmo/model.py:516-531): slice, cast to the activation dtype,
            # replace -inf by the dtype's minimum.
            bias = bias[:, :, L - T : L, :L]
            if bias.dtype != self.act:
                bias = bias.to(self.act)
                bias = bias.masked_fill(bias == float("-inf"), _finfo_min(self.act))
        att = attention(q, k, v, bias, self.act)
        att = att.transpose(1, 2).contiguous().view(B, T, C)
        return self.linear(pre + "attn_out", att), present

    def _block(self, i, x, bias, layer_past, use_cache):
        c = self.cfg
        pre = f"transformer.blocks.{i}."
        hd = c.d_model // c.n_heads
        h = x if c.norm_after else self._norm(pre + "attn_norm", x)
        qkv = self.linear(pre + "att_proj", h)
        if c.clip_qkv is not None:  # olmo/model.py:756-757
            qkv = qkv.clamp(min=-c.clip_qkv, max=c.clip_qkv)
        dkv = c.effective_n_kv_heads * hd
        q, k, v = qkv.split((c.d_model, dkv, dkv), dim=-1)
        att, cache = self._attention(i, q, k, v, bias, layer_past, use_cache)
        if c.norm_after:
            att = self._norm(pre + "attn_norm", att)
        x = x + att
        og = x
        if not c.norm_after:
            x = self._norm(pre + "ff_norm", x)
        x = self.linear(pre + "ff_proj", x)
        x = swiglu(x)
        x = self.linear(pre + "ff_out", x)
        if c.norm_after:
            x = self._norm(pre + "ff_norm", x)
        return og + x, cache

    # -- whole forward ---------------------------------------------------------------------
    @torch.no_grad()
    def forward(
        self,
        input_ids: torch.Tensor,
        attention_mask: Optional[torch.Tensor] = None,
        past_key_values: Optional[Sequence[Tuple[torch.Tensor, torch.Tensor]]] = None,
        use_cache: bool = False,
        last_logits_only: bool = False,
        attention_bias: Optional[torch.Tensor] = None,
    ) -> Tuple[torch.Tensor, Optional[List[Tuple[torch.Tensor, torch.Tensor]]]]:
        c = self.cfg
        B, T = input_ids.shape
        past_len = 0 if past_key_values is None else past_key_values[0][0].size(-2)
        x = self.w["transformer.wte.weight"].to(self.act)[input_ids]

        bias = None
        if attention_mask is not None:
            am = attention_mask.to(torch.float).view(B, -1)[:, None, None, :]
            am = (1.0 - am) * _finfo_min(torch.float)
        else:
            am = None
        if am is not None or past_key_values is not None or attention_bias is not None:
            # olmo/model.py:1343-1376 with causal_attention_bias (:375-381); an explicit bias replaces the
            # causal one, and a bool / int8 one is turned into 1.0 / most-negative first (:1358-1360)
            L = past_len + T
            if attention_bias is None:
                bias = torch.triu(torch.ones(L, L, dtype=torch.float), diagonal=1)
                bias = bias.masked_fill(bias == 1, _finfo_min(torch.float)).view(1, 1, L, L)
            elif attention_bias.dtype in (torch.int8, torch.bool):
                bias = attention_bias.to(torch.float)
                bias = bias.masked_fill(bias == 0.0, _finfo_min(torch.float))
            else:
                bias = attention_bias
            mask_len = am.shape[-1] if am is not None else L
            bias = bias.to(torch.float)
            bias = bias[:, :, :mask_len, :mask_len]
            if am is not None:
                bias = bias + am
                bias = bias.masked_fill(bias == float("-inf"), _finfo_min(torch.float))

        kvs: Optional[List] = [] if use_cache else None
        for i in range(c.n_layers):
            lp = None if past_key_values is None else past_key_values[i]
            x, cache = self._block(i, x, bias, lp, use_cache)
            if kvs is not None:
                kvs.append(cache)
        if last_logits_only:
            x = x[:, -1, :].unsqueeze(1)
        x = self._norm("transformer.ln_f", x)
        # weight tying: the embedding is the output matrix (olmo/model.py:1454-1457)
        logits = self.linear("transformer.wte" if c.weight_tying else "transformer.ff_out", x)
        return logits, kvs


def random_weights(cfg, dtype: torch.dtype, seed: int = 0, quantized: bool = False, group_size: int = 128,
                   norm_weight_std: float = 0.0) -> Dict[str, torch.Tensor]:
    """Synthetic weights of the reference's shapes: Linear / embedding weights N(0, init_std)
    (``olmo/initialization.py:8-22`` fixes the distribution), norm weights 1 (optionally
    perturbed), and, when ``quantized``, the four block Linears as random int4 buffers."""
    gen = torch.Generator().manual_seed(seed)
    hd = cfg.d_model // cfg.n_heads
    dkv = cfg.effective_n_kv_heads * hd
    w: Dict[str, torch.Tensor] = {}

    def normal(*shape):
        return (torch.randn(*shape, generator=gen) * cfg.init_std).to(dtype)

    def normw(n):
        t = torch.ones(n)
        if norm_weight_std:
            t = t + torch.randn(n, generator=gen) * norm_weight_std
        return t.to(dtype)

    hidden = cfg.mlp_hidden_size if cfg.mlp_hidden_size is not None else cfg.mlp_ratio * cfg.d_model
    w["transformer.wte.weight"] = normal(cfg.embedding_size or cfg.vocab_size, cfg.d_model)
    for i in range(cfg.n_layers):
        pre = f"transformer.blocks.{i}."
        shapes = {
            "att_proj": (cfg.d_model + 2 * dkv, cfg.d_model),
            "attn_out": (cfg.d_model, cfg.d_model),
            "ff_proj": (hidden, cfg.d_model),
            "ff_out": (cfg.d_model, hidden // 2),
        }
        for name, (N, K) in shapes.items():
            if quantized:
                s = int(torch.randint(0, 2**31 - 1, (1,), generator=gen))
                qw, qz, sc = w4.random_quantized(K, N, group_size, seed=s)
                w[pre + name + ".qweight"], w[pre + name + ".qzeros"], w[pre + name + ".scales"] = qw, qz, sc
            else:
                w[pre + name + ".weight"] = normal(N, K)
        if cfg.layer_norm_type == "rms":
            w[pre + "attn_norm.weight"] = normw(cfg.d_model)
            w[pre + "ff_norm.weight"] = normw(cfg.d_model)
            if cfg.attention_layer_norm:
                w[pre + "q_norm.weight"] = normw(cfg.d_model)
                w[pre + "k_norm.weight"] = normw(dkv)
    if cfg.layer_norm_type == "rms":
        w["transformer.ln_f.weight"] = normw(cfg.d_model)
    if not cfg.weight_tying:  # olmo/model.py:1129-1137: no separate output matrix when tied
        w["transformer.ff_out.weight"] = normal(cfg.embedding_size or cfg.vocab_size, cfg.d_model)
    return w
