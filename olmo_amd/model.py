"""``OLMo``: the reference's inference forward pass on one MI355X, computed by the HIP kernels
of this package.

Drop-in for ``olmo/model.py``'s ``OLMo.forward`` (``:1253-1465``): same arguments, same
``OLMoOutput`` tuple, same module tree / parameter names (``transformer.wte``,
``transformer.blocks.{i}.att_proj`` ... ``transformer.ln_f``, ``transformer.ff_out``) so that a
reference state dict loads by name and AutoGPTQ-style ``make_quant`` can swap the block
Linears.  PyTorch holds the parameters and device buffers; every arithmetic step is a kernel
call through the C-ABI (``olmo_amd.ops``).

KV cache.  The reference returns per layer ``(k, v)`` of shape ``[B, n_kv_heads, L, hd]`` with
``k`` *before* rotary embedding and re-rotates the whole cache each step
(``olmo/model.py:615-625``).  Here each layer owns one contiguous buffer of capacity
``max_cache_len`` holding the *rotated* keys; ``attn_key_values`` are ``LayerKV`` tuples of
views ``[:, :, :L]`` into it.  Passing them back as ``past_key_values`` continues in place with
no copy.  Plain tensors passed as ``past_key_values`` are taken to be in the reference's
form and are rotated into a fresh cache first.
"""

from __future__ import annotations

import math
from typing import Dict, List, NamedTuple, Optional, Sequence, Tuple

import torch
import torch.nn as nn

from . import ops
from .config import ModelConfig, OLMoConfigurationError
from .qlinear import QuantLinear

__all__ = ["OLMo", "OLMoOutput", "OLMoGenerateOutput", "LayerKV", "KVCache", "DenseLinear"]


class OLMoOutput(NamedTuple):
    """``olmo/model.py:980-995``."""

    logits: torch.Tensor
    attn_key_values: Optional[List[Tuple[torch.Tensor, torch.Tensor]]]
    hidden_states: Optional[Tuple[torch.Tensor, ...]]


class OLMoGenerateOutput(NamedTuple):
    """``olmo/model.py:998-1009``: ``token_ids [B, beam, steps]``, ``scores [B, beam]``."""

    token_ids: torch.Tensor
    scores: torch.Tensor


class KVCache:
    """Contiguous per-layer key/value buffers ``[B, n_kv_heads, capacity, hd]`` (keys rotated)."""

    def __init__(self, n_layers: int, B: int, Hkv: int, capacity: int, hd: int, dtype, device):
        # one allocation for all layers (a fresh cache is made per prompt: 2 * n_layers separate ones cost a 7B
        # prefill 2.9 ms of allocator calls when none of them was cached); a layer's keys and values are the
        # contiguous slices [B, Hkv, capacity, hd] of it
        kv = torch.empty(2, n_layers, B, Hkv, capacity, hd, dtype=dtype, device=device)
        self.k = list(kv[0].unbind(0))
        self.v = list(kv[1].unbind(0))
        self.B, self.capacity, self.length = B, capacity, 0
        # device copy of the number of cached positions, for captured decode steps
        self.length_dev = torch.zeros(1, dtype=torch.int32, device=device)
        # rotary rows [sin | cos] of position `length`, kept current by a decode session (None otherwise)
        self.rope_now: Optional[torch.Tensor] = None

    def views(self) -> List["LayerKV"]:
        L = self.length
        return [LayerKV((k[:, :, :L], v[:, :, :L]), self) for k, v in zip(self.k, self.v)]

    def set_length(self, L: int) -> None:
        self.length = L
        self.length_dev.fill_(L)


class BeamKVCache(KVCache):
    """Cache of a beam search: row ``b`` is beam ``b % beam`` of sequence ``b // beam``.  The prompt's keys and
    values live once per sequence, in the row of its first beam; generated token ``i`` of a beam's history lives
    in row ``beam_src[b, i]``, the row of the beam that fed it.  Choosing parents (``reorder_beams``) rewrites
    that small table; no cache row is ever copied, where ``olmo/beam_search.py:1062-1078`` gathers all
    ``2 * n_layers`` cache tensors after every step."""

    def __init__(self, n_layers: int, B: int, beam: int, Hkv: int, prompt_len: int, steps: int, hd: int, dtype, device):
        super().__init__(n_layers, B * beam, Hkv, prompt_len + steps, hd, dtype, device)
        self.beam, self.prompt_len = beam, prompt_len
        self._own = torch.arange(B * beam, dtype=torch.int32, device=device).unsqueeze(1)
        self.beam_src = self._own.expand(B * beam, steps).contiguous()
        self._seq0 = (torch.arange(B, device=device) * beam).unsqueeze(1)

    def reorder_beams(self, backpointer: torch.Tensor) -> None:
        rows = (backpointer.to(self._seq0.device) + self._seq0).reshape(-1)
        src = self.beam_src.index_select(0, rows)
        written = self.length - self.prompt_len  # generated tokens already in the cache
        src[:, written:] = self._own            # whatever a beam feeds next goes to its own row
        self.beam_src.copy_(src)                # in place: a captured step keeps reading the same table


class LayerKV(tuple):
    """``(k, v)`` views of one layer's cache, remembering the cache they belong to."""

    def __new__(cls, kv, cache: KVCache):
        self = super().__new__(cls, kv)
        self.cache = cache
        return self


class DenseLinear(nn.Linear):
    """``nn.Linear`` without bias whose product runs on the HIP kernels (bf16, fp16: re-tiled copy on
    the matrix cores; fp32: FMA kernel).  Parameters are left uninitialised: weights come from a
    state dict or from ``OLMo.reset_parameters``."""

    def __init__(self, in_features: int, out_features: int, device=None, dtype=None):
        nn.Module.__init__(self)
        self.in_features, self.out_features = in_features, out_features
        self.weight = nn.Parameter(torch.empty(out_features, in_features, device=device, dtype=dtype),
                                   requires_grad=False)
        self.register_parameter("bias", None)
        self._tiled: Optional[ops.B16Tiled] = None

    def reset_parameters(self) -> None:  # nn.Linear's default init is not wanted
        pass

    def post_init(self):
        if self.weight.dtype in (torch.bfloat16, torch.float16):
            self._tiled = ops.b16_repack(self.weight.data.contiguous())
        return self

    def tiled_weight(self) -> ops.B16Tiled:
        if self._tiled is None:
            self.post_init()
        return self._tiled

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.weight.dtype == torch.float32:
            return ops.f32_linear(x, self.weight.data)
        return ops.b16_linear(x, self.tiled_weight())


class RMSLayerNorm(nn.Module):
    """``olmo/model.py:228-255``; parameter name ``weight`` as in the reference."""

    def __init__(self, size: int, eps: float, device=None, dtype=None):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(size, device=device, dtype=dtype), requires_grad=False)

    def forward(self, x, residual=None):
        return ops.rmsnorm(x, self.weight.data, self.eps, residual=residual)


class LayerNormNP(nn.Module):
    """Non-parametric ``LayerNorm`` (``olmo/model.py:193-225`` with ``elementwise_affine=False``)."""

    def __init__(self, size: int, eps: float):
        super().__init__()
        self.eps = eps
        self.weight = None

    def forward(self, x, residual=None):
        y = ops.layernorm_np(x, self.eps)
        return y if residual is None else ops.add(residual, y)


def _build_norm(cfg: ModelConfig, size: int, device, dtype) -> nn.Module:
    if cfg.layer_norm_type == "rms":
        return RMSLayerNorm(size, cfg.layer_norm_eps, device, dtype)
    return LayerNormNP(size, cfg.layer_norm_eps)


class OLMoSequentialBlock(nn.Module):
    """Module set of ``olmo/model.py:396-506,685-705``; the arithmetic is in ``OLMo._block``."""

    def __init__(self, layer_id: int, cfg: ModelConfig, device, dtype, weight_device=None):
        super().__init__()
        self.layer_id = layer_id
        hd = cfg.head_dim
        dkv = cfg.effective_n_kv_heads * hd
        wdev = weight_device if weight_device is not None else device
        self.att_proj = DenseLinear(cfg.d_model, cfg.d_model + 2 * dkv, wdev, dtype)
        self.attn_out = DenseLinear(cfg.d_model, cfg.d_model, wdev, dtype)
        self.ff_proj = DenseLinear(cfg.d_model, cfg.hidden_size, wdev, dtype)
        self.ff_out = DenseLinear(cfg.act_out_size, cfg.d_model, wdev, dtype)
        self.attn_norm = _build_norm(cfg, cfg.d_model, device, dtype)
        self.ff_norm = _build_norm(cfg, cfg.d_model, device, dtype)
        if cfg.attention_layer_norm:
            self.q_norm = RMSLayerNorm(cfg.d_model, cfg.layer_norm_eps, device, dtype)
            self.k_norm = RMSLayerNorm(dkv, cfg.layer_norm_eps, device, dtype)
        else:
            self.q_norm = self.k_norm = None


class _Embedding(nn.Module):
    def __init__(self, n: int, d: int, device, dtype):
        super().__init__()
        self.weight = nn.Parameter(torch.empty(n, d, device=device, dtype=dtype), requires_grad=False)

    def forward(self, ids):
        return ops.embedding(ids.contiguous(), self.weight.data)


RELAY = False             # opt-in: the one-row decode step as a two-stream relay (measured: not faster than the chained step)
RELAY_TWO_STREAMS = True  # ... or keep it on one stream inside a captured step
RELAY_FENCE = ()           # tuning: launches fenced off from the other stream ("pre:attention", "post:ff_out", ...)


class _RelayState:
    """Buffers, epoch and launch plan of the one-row decode relay (``olmo_amd/csrc/relay.hip``): every tensor that
    passes from one launch of a step to the next lives here, one per block and role, each written exactly once per
    step -- which is what lets a launch on the second stream start before its producer has finished."""

    # launch shapes tried per linear, in order of preference (0 = the kernel's own choice; waves | tiles << 8)
    CANDIDATES = {"att_proj": (0, 8 | 2 << 8, 16 | 2 << 8), "attn_out": (0, 8 | 1 << 8), "ff_proj": (0, 16 | 2 << 8),
                  "ff_out": (0, 8 | 1 << 8)}

    def __init__(self, model: "OLMo"):
        c, dev = model.config, model.device
        d, dkv = c.d_model, c.effective_n_kv_heads * c.head_dim
        width, h2 = d + 2 * dkv, c.act_out_size
        i32 = lambda n: torch.zeros(n, dtype=torch.int32, device=dev)
        self.epoch, self.status = i32(1), i32(8)  # status: [0] a wait gave up; [1..3] wait statistics when [4] is set
        self.x0 = i32(d)  # the token's embedding, tagged: the first residual row
        self.layers = [dict(qkv=i32(width), ssq_qkv=i32(width // 16), att=i32(d), a=i32(d), ssq_a=i32(d // 16), x1=i32(d),
                            u=i32(h2), x2=i32(d), f=i32(d), ssq_f=i32(d // 16)) for _ in range(c.n_layers)]
        # per launch: 64 copies, 1 KiB apart, of a word set to the epoch when the launch's last workgroup is done
        self.hints = torch.zeros(c.n_layers * 5, 64 * 256, dtype=torch.int32, device=dev)
        self.side = torch.cuda.Stream(device=dev)
        self.shapes = {"att_proj": (width, d, True, False), "attn_out": (d, d, False, False),
                       "ff_proj": (c.hidden_size, d, True, True), "ff_out": (d, h2, False, False)}  # N, K, norm, swiglu
        self.cfg = {k: 0 for k in self.shapes}
        self.plans: Dict[int, Optional[Dict[str, int]]] = {}
        self.attn_ok: Dict[int, bool] = {}
        self.covered = all(ops.relay_footprint_w4(n, k, nm, sw) is not None for n, k, nm, sw in self.shapes.values()) \
            and c.head_dim in (64, 128) and d <= 8192 and dkv <= 8192

    def plan(self, model: "OLMo", n_keys_max: int) -> Optional[Dict[str, int]]:
        """Launch shapes under which every pair of consecutive launches of a step fits the chip side by side (the
        condition for running them on two streams), or ``None`` when there is no such choice."""
        if n_keys_max in self.plans:
            return self.plans[n_keys_max]
        import itertools

        c = model.config
        n_cu, lds = ops.relay_device()
        att = ops.relay_footprint_attn(c.n_heads, c.head_dim, n_keys_max)
        found = None
        if att is not None:
            names = ("att_proj", "attn_out", "ff_proj", "ff_out")
            for combo in itertools.product(*(self.CANDIDATES[n] for n in names)):
                fp = {}
                for n, cf in zip(names, combo):
                    N, K, nm, sw = self.shapes[n]
                    fp[n] = ops.relay_footprint_w4(N, K, nm, sw, cf)
                if any(v is None for v in fp.values()):
                    continue
                order = [fp["att_proj"], att, fp["attn_out"], fp["ff_proj"], fp["ff_out"]]
                if all(ops.relay_pair_ok(order[i], order[(i + 1) % 5], n_cu, lds) for i in range(5)):
                    found = dict(zip(names, combo))
                    break
        self.plans[n_keys_max] = found
        return found


class OLMo(nn.Module):
    def __init__(self, config: ModelConfig, device="cuda", dtype: torch.dtype = torch.bfloat16,
                 max_cache_len: Optional[int] = None, block_weight_device=None):
        """``block_weight_device='meta'`` leaves the four dense Linears of every block unallocated
        (for models whose block Linears are about to be replaced by ``QuantLinear``)."""
        super().__init__()
        config.validate_for_inference()
        if dtype not in (torch.bfloat16, torch.float16, torch.float32):
            raise OLMoConfigurationError("activation dtype must be bfloat16, float16 or float32")
        self.config = config
        self.device = torch.device(device)
        self.dtype = dtype
        self.max_cache_len = max_cache_len or config.max_sequence_length
        V = config.logits_size
        self.transformer = nn.ModuleDict(dict(
            wte=_Embedding(V, config.d_model, device, dtype),
            blocks=nn.ModuleList([OLMoSequentialBlock(i, config, device, dtype, block_weight_device)
                                  for i in range(config.n_layers)]),
            ln_f=_build_norm(config, config.d_model, device, dtype),
        ))
        if not config.weight_tying:  # olmo/model.py:1129-1137
            self.transformer.update({"ff_out": DenseLinear(config.d_model, V, device, dtype)})
        self._tied_head: Optional[ops.B16Tiled] = None  # weight tying, 16-bit: the embedding re-tiled as the output matrix
        self._prepared = False
        self._act_order = False
        self._rope: Optional[Tuple[torch.Tensor, torch.Tensor]] = None
        self._attn_ws: Dict[Tuple[int, int], torch.Tensor] = {}
        self._scratch_kv: Dict[Tuple[int, int], Tuple[torch.Tensor, torch.Tensor]] = {}

    # ------------------------------------------------------------------------------------------
    # parameters
    # ------------------------------------------------------------------------------------------
    @torch.no_grad()
    def reset_parameters(self, seed: int = 0) -> None:
        """Linear and embedding weights ~ N(0, init_std), truncated at ``init_cutoff_factor`` sigmas
        when set (``olmo/initialization.py:8-22``); norm weights 1.  (The reference's parameter
        visiting order, hence its exact random stream, is not reproduced.)"""
        gen = torch.Generator(device=self.device).manual_seed(seed)
        c = self.config
        for p in self.parameters():
            if p.device.type == "meta":
                continue
            if p.dim() == 1:
                p.fill_(1.0)
            else:
                t = torch.empty(p.shape, dtype=torch.float32, device=self.device).normal_(0.0, c.init_std, generator=gen)
                if c.init_cutoff_factor:
                    t.clamp_(-c.init_cutoff_factor * c.init_std, c.init_cutoff_factor * c.init_std)
                p.copy_(t.to(p.dtype))
        self._prepared = False

    def post_init(self) -> "OLMo":
        """Build the kernel-side weight layouts, rotary tables (idempotent)."""
        # a loader that swaps parameters in (transformers' ``from_pretrained`` without a device map leaves them in
        # host memory) is followed here: everything the kernels read lives on this model's GPU
        if any(t.device.type not in (self.device.type, "meta") for t in list(self.parameters()) + list(self.buffers())):
            self.to(self.device)
        for m in self.modules():
            if isinstance(m, (DenseLinear, QuantLinear)) and m is not self:
                if isinstance(m, DenseLinear) and m.weight.device.type == "meta":
                    raise RuntimeError("a block Linear is still on the meta device: swap it or load weights first")
                m.post_init()
        c = self.config
        if c.weight_tying and self.dtype != torch.float32:
            self._tied_head = ops.b16_repack(self.transformer["wte"].weight.data.contiguous())
        n_pos = max(self.max_cache_len, c.max_sequence_length)
        self._rope = ops.rope_tables(c.head_dim, float(c.rope_theta), n_pos, self.device)
        # act-order int4 layers gather their activation columns in QuantLinear.forward, which also adds a
        # non-zero bias: the fused decode forms (which hand the tiled weights to the kernels directly) are
        # not used for such models
        self._act_order = any(isinstance(m, QuantLinear) and (m._perm is not None or m._has_bias) for m in self.modules())
        self._chain_ok = {}  # rows -> whether the chained decode block covers this model
        self._relay: Optional[_RelayState] = None  # state of the one-row decode relay, made on first use
        self._rope_now = None  # rotary rows of the current position during a captured decode step
        self._beam = None  # the beam cache while a beam-search step runs
        self._prepared = True
        return self

    def load_reference_state_dict(self, sd: Dict[str, torch.Tensor]) -> None:
        """Load tensors keyed by the reference's names (``transformer....``); int4 buffers go to
        ``QuantLinear`` modules, dense weights are cast to the model dtype."""
        own = dict(self.named_parameters())
        own.update(dict(self.named_buffers()))
        missing = []
        with torch.no_grad():
            for name, tgt in own.items():
                if tgt.device.type == "meta":
                    continue
                if name not in sd:
                    if not name.endswith((".g_idx", ".bias")):
                        missing.append(name)
                    continue
                src = sd[name]
                if tuple(src.shape) != tuple(tgt.shape):
                    raise ValueError(f"{name}: shape {tuple(src.shape)} != {tuple(tgt.shape)}")
                tgt.copy_(src.to(device=tgt.device, dtype=tgt.dtype))
        if missing:
            raise KeyError(f"missing tensors: {missing[:5]}{'...' if len(missing) > 5 else ''}")
        for m in self.modules():
            if isinstance(m, QuantLinear):
                m._tiled = None
        self._prepared = False

    # ------------------------------------------------------------------------------------------
    # cache handling
    # ------------------------------------------------------------------------------------------
    def new_cache(self, B: int, capacity: Optional[int] = None) -> KVCache:
        c = self.config
        return KVCache(c.n_layers, B, c.effective_n_kv_heads, capacity or self.max_cache_len, c.head_dim, self.dtype,
                       self.device)

    def _ingest_reference_cache(self, past: Sequence[Tuple[torch.Tensor, torch.Tensor]], new_tokens: int) -> KVCache:
        """Reference-form ``past_key_values`` (keys not rotated) -> a cache of this model."""
        c = self.config
        B, Hkv, L, hd = past[0][0].shape
        cache = self.new_cache(B, max(self.max_cache_len, L + new_tokens))
        sin, cos = self._rope
        for i, (k, v) in enumerate(past):
            # reuse the rotary kernel: feed [q | k | v] rows with q := k (discarded), no norm
            kt = k.to(self.device, self.dtype).transpose(1, 2).reshape(B * L, Hkv * hd)
            vt = v.to(self.device, self.dtype).transpose(1, 2).reshape(B * L, Hkv * hd)
            qkv = torch.cat((kt, kt, vt), dim=-1).contiguous()
            ops.qknorm_rope_kvwrite(qkv, None, None, sin, cos, cache.k[i], cache.v[i], B, L, Hkv, Hkv, hd, 0,
                                    c.layer_norm_eps)
        cache.set_length(L)
        return cache

    def _scratch_cache(self, B: int, T: int):
        key = (B, T)
        if key not in self._scratch_kv:
            self._scratch_kv.clear()
            c = self.config
            shape = (B, c.effective_n_kv_heads, T, c.head_dim)
            self._scratch_kv[key] = (torch.empty(shape, dtype=self.dtype, device=self.device),
                                     torch.empty(shape, dtype=self.dtype, device=self.device))
        return self._scratch_kv[key]

    def _decode_ws(self, B: int, n_keys_max: int) -> torch.Tensor:
        """Attention workspace for ``B`` rows and up to ``n_keys_max`` keys, sized in steps of 1024 keys so that
        eager decoding (a new key count every step) reuses one buffer instead of allocating one per length."""
        key = (B, -(-n_keys_max // 1024) * 1024)
        if key not in self._attn_ws:
            c = self.config
            self._attn_ws[key] = ops.attn_decode_workspace(B, c.n_heads, c.head_dim, key[1], self.device)
        return self._attn_ws[key]

    # ------------------------------------------------------------------------------------------
    # one block: olmo/model.py:728-823 (wiring), :588-654 (attention)
    # ------------------------------------------------------------------------------------------
    def _linear(self, m: nn.Module, x: torch.Tensor) -> torch.Tensor:
        return m(x)

    def _attention(self, blk, qkv, kc, vc, B, T, past_len, key_bias, graph_pos, n_keys_max, qk_ssq=None):
        c = self.config
        H, Hkv, hd = c.n_heads, c.effective_n_kv_heads, c.head_dim
        sin, cos = self._rope
        qw = blk.q_norm.weight.data if blk.q_norm is not None else None
        kw = blk.k_norm.weight.data if blk.k_norm is not None else None
        decode = T == 1 and (graph_pos is not None or past_len > 0)
        beam = self._beam
        if decode and beam is None:
            att = ops.attn_decode_fused(qkv, qw, kw, sin, cos, kc, vc, self._decode_ws(B, n_keys_max), B, H, Hkv, hd,
                                        past_len, n_keys_max, c.layer_norm_eps, key_bias=key_bias,
                                        past_len_dev=graph_pos, qk_ssq=qk_ssq,
                                        rope_now=self._rope_now if graph_pos is not None else None)
            if att is not None:
                return att
        q = ops.qknorm_rope_kvwrite(qkv, qw, kw, sin, cos, kc, vc, B, T, H, Hkv, hd, past_len, c.layer_norm_eps,
                                    past_len_dev=graph_pos)
        if decode:
            if beam is not None:
                return ops.attn_decode(q, kc, vc, self._decode_ws(B, n_keys_max), B, H, Hkv, hd, past_len, n_keys_max,
                                       key_bias=key_bias, past_len_dev=graph_pos, beam_src=beam.beam_src,
                                       prompt_len=beam.prompt_len, beam=beam.beam)
            return ops.attn_decode(q, kc, vc, self._decode_ws(B, n_keys_max), B, H, Hkv, hd, past_len, n_keys_max,
                                   key_bias=key_bias, past_len_dev=graph_pos)
        return ops.attn_prefill(q, kc, vc, B, T, H, Hkv, hd, past_len, key_bias=key_bias)

    def _block(self, blk: OLMoSequentialBlock, x, kc, vc, B, T, past_len, key_bias, graph_pos, n_keys_max):
        c = self.config
        h = x if c.norm_after else blk.attn_norm(x)
        qkv = self._linear(blk.att_proj, h)
        if c.clip_qkv is not None:
            ops.clamp_(qkv, c.clip_qkv)
        att = self._attention(blk, qkv, kc, vc, B, T, past_len, key_bias, graph_pos, n_keys_max)
        att = self._linear(blk.attn_out, att)
        x = blk.attn_norm(att, residual=x) if c.norm_after else ops.add(x, att)
        h = x if c.norm_after else blk.ff_norm(x)
        rows = B * T
        if (self.dtype == torch.bfloat16 and not self._act_order
                and (rows <= 16 or (rows > ops.GEMV_MAX_M and isinstance(blk.ff_proj, QuantLinear)))):
            # SwiGLU rides in the projection's epilogue (few rows: the GEMV's; many rows: the int4 GEMM's)
            h, _ = ops.linear_fused(h, self._tiled(blk.ff_proj), swiglu_out=True)
        else:
            h = ops.swiglu(self._linear(blk.ff_proj, h))
        h = self._linear(blk.ff_out, h)
        return blk.ff_norm(h, residual=x) if c.norm_after else ops.add(x, h)

    # Decode form of the OLMo-2 (post-norm, RMS) block with the residual/norm updates folded into the
    # linear that consumes them and SwiGLU into ff_proj: 6 launches per layer instead of 10.
    #   x      residual stream entering the block, *before* the previous block's pending update
    #   pend   (f_prev, ff_norm weight of the previous block) or None: x := x + norm(f_prev) is applied
    #          inside this block's att_proj launch
    def _fused_decode_ok(self, M: int, collect_hidden: bool, rows_in_lds: bool = True) -> bool:
        """Whether a decode step of ``M`` rows may fold the norms into its linears.  ``rows_in_lds``: for the kernels
        that keep all rows of the activations in LDS (the chained form for 5 to 8 rows does not)."""
        c = self.config
        ok = (M <= 16 and self.dtype == torch.bfloat16 and c.norm_after and c.layer_norm_type == "rms"
              and not collect_hidden and not self._act_order and c.clip_qkv is None)
        if rows_in_lds:
            ok = ok and c.d_model * 2 * (M + 1) <= 64 * 1024 and c.d_model <= 5120
        return ok

    @staticmethod
    def _tiled(m: nn.Module):
        return m.tiled if isinstance(m, QuantLinear) else m.tiled_weight()

    def _block_decode_fused(self, blk, x, pend, kc, vc, B, past_len, key_bias, graph_pos, n_keys_max):
        eps = self.config.layer_norm_eps
        if pend is None:
            qkv = self._linear(blk.att_proj, x)
        else:
            # x := x + norm(previous block's MLP output) happens in the projection's prologue
            qkv, x = ops.linear_fused(pend[0], self._tiled(blk.att_proj), resid=x, norm_w=pend[1], eps=eps)
        att = self._attention(blk, qkv, kc, vc, B, 1, past_len, key_bias, graph_pos, n_keys_max)
        a = self._linear(blk.attn_out, att)
        u, x = ops.linear_fused(a, self._tiled(blk.ff_proj), resid=x, norm_w=blk.attn_norm.weight.data, eps=eps,
                                swiglu_out=True)
        f = self._linear(blk.ff_out, u)
        return x, (f, blk.ff_norm.weight.data)

    # The same block for at most 4 rows of int4 weights, with the three norms *chained*: the launch that
    # produces a tensor also leaves the sums of squares of its 16-column tiles, and the launch that
    # normalises the tensor (att_proj / ff_proj prologue, QK-norm inside attention) adds those up instead
    # of re-reading the row and synchronising its workgroup.
    #   pend   (f_prev, ff_norm weight, ssq of f_prev) or None
    def _block_decode_chain(self, blk, x, pend, kc, vc, B, past_len, key_bias, graph_pos, n_keys_max):
        eps = self.config.layer_norm_eps
        qknorm = blk.q_norm is not None
        if pend is None:
            qkv, _, ssq_qkv = ops.w4_linear_chain(x, blk.att_proj.tiled, want_ssq=qknorm)
        else:
            qkv, x, ssq_qkv = ops.w4_linear_chain(pend[0], blk.att_proj.tiled, resid=x, norm_w=pend[1], eps=eps,
                                                  ssq_in=pend[2], want_ssq=qknorm)
        att = self._attention(blk, qkv, kc, vc, B, 1, past_len, key_bias, graph_pos, n_keys_max, qk_ssq=ssq_qkv)
        a, _, ssq_a = ops.w4_linear_chain(att, blk.attn_out.tiled, want_ssq=True)
        u, x, _ = ops.w4_linear_chain(a, blk.ff_proj.tiled, resid=x, norm_w=blk.attn_norm.weight.data, eps=eps,
                                      ssq_in=ssq_a, swiglu_out=True)
        f, _, ssq_f = ops.w4_linear_chain(u, blk.ff_out.tiled, want_ssq=True)
        return x, (f, blk.ff_norm.weight.data, ssq_f)

    # The one-row decode step as a relay (olmo_amd/csrc/relay.hip): the chained block above with every hand-over
    # between launches carried by epoch tags in the data.  On one stream this is the same arithmetic launch for launch;
    # inside a captured step the launches alternate between two streams, so that each one requests its weights while
    # its predecessor still computes.  Returns the residual row after the last block (bf16 [1, 1, d]).
    def _relay_blocks(self, x, cache: KVCache, past_len: int, key_bias, graph_pos, n_keys_max: int) -> torch.Tensor:
        c, rs = self.config, self._relay
        eps = c.layer_norm_eps
        H, Hkv, hd = c.n_heads, c.effective_n_kv_heads, c.head_dim
        sin, cos = self._rope
        ws = self._decode_ws(1, n_keys_max)
        main = torch.cuda.current_stream()
        # two streams only inside a captured step (eager launches are bound by the host anyway), with the plan made
        # beforehand (planning queries kernel attributes, which has no place inside a capture)
        plan = rs.plans.get(n_keys_max) if (RELAY_TWO_STREAMS and torch.cuda.is_current_stream_capturing()) else None
        cfg = plan if plan is not None else rs.cfg
        ops.incr_i32(rs.epoch)
        ops.relay_tag(x.view(-1), rs.x0, rs.epoch)
        if plan is not None:
            rs.side.wait_stream(main)
            lanes = (main.cuda_stream, rs.side.cuda_stream)
        else:
            lanes = (main.cuda_stream, main.cuda_stream)
        n = 0  # launches so far: launch n goes to stream n % 2
        streams = (main, rs.side)

        def fence(which):  # tuning knob: keep the named launch apart from its neighbours on the other stream
            if plan is not None and which in RELAY_FENCE:
                streams[0].wait_stream(streams[1])
                streams[1].wait_stream(streams[0])

        # hint words only where a launch may run beside its producer: without one a launch asks for its rows at once
        hint = lambda i: dict(hint_in=rs.hints[i - 1] if (i > 0 and plan is not None) else None, hint_out=rs.hints[i] if plan is not None else None)
        resid, pend = rs.x0, None
        rope_now = self._rope_now if graph_pos is not None else None
        for blk, L in zip(self.transformer["blocks"], rs.layers):
            qknorm = blk.q_norm is not None
            ssq_qkv = L["ssq_qkv"] if qknorm else None
            fence("pre:att_proj")
            if pend is None:
                ok = ops.w4_relay(rs.x0, blk.att_proj.tiled, L["qkv"], rs.epoch, rs.status, ssq_out=ssq_qkv,
                                  cfg=cfg["att_proj"], stream=lanes[n % 2], **hint(n))
            else:
                ok = ops.w4_relay(pend[0], blk.att_proj.tiled, L["qkv"], rs.epoch, rs.status, resid=resid, norm_w=pend[1],
                                  eps=eps, ssq_in=pend[2], x_out=L["x1"], ssq_out=ssq_qkv, cfg=cfg["att_proj"],
                                  stream=lanes[n % 2], **hint(n))
                resid = L["x1"]
            n += 1
            fence("post:att_proj"), fence("pre:attention")
            ok = ok and ops.attn_decode_relay(L["qkv"], blk.q_norm.weight.data if qknorm else None,
                                              blk.k_norm.weight.data if qknorm else None, sin, cos, cache.k[blk.layer_id],
                                              cache.v[blk.layer_id], ws, L["att"], H, Hkv, hd, past_len, n_keys_max, eps,
                                              rs.epoch, rs.status, key_bias=key_bias, past_len_dev=graph_pos, qk_ssq=ssq_qkv,
                                              rope_now=rope_now, stream=lanes[n % 2], **hint(n))
            n += 1
            fence("post:attention"), fence("pre:attn_out")
            ok = ok and ops.w4_relay(L["att"], blk.attn_out.tiled, L["a"], rs.epoch, rs.status, ssq_out=L["ssq_a"],
                                     cfg=cfg["attn_out"], stream=lanes[n % 2], **hint(n))
            n += 1
            fence("post:attn_out"), fence("pre:ff_proj")
            ok = ok and ops.w4_relay(L["a"], blk.ff_proj.tiled, L["u"], rs.epoch, rs.status, resid=resid,
                                     norm_w=blk.attn_norm.weight.data, eps=eps, ssq_in=L["ssq_a"], x_out=L["x2"], swiglu=True,
                                     cfg=cfg["ff_proj"], stream=lanes[n % 2], **hint(n))
            resid = L["x2"]
            n += 1
            fence("post:ff_proj"), fence("pre:ff_out")
            ok = ok and ops.w4_relay(L["u"], blk.ff_out.tiled, L["f"], rs.epoch, rs.status, ssq_out=L["ssq_f"],
                                     cfg=cfg["ff_out"], stream=lanes[n % 2], **hint(n))
            n += 1
            fence("post:ff_out")
            if not ok:
                raise RuntimeError("the decode relay declined a launch it had accepted when it was planned")
            pend = (L["f"], blk.ff_norm.weight.data, L["ssq_f"])
        if plan is not None:
            main.wait_stream(rs.side)
        out = torch.empty(1, 1, c.d_model, dtype=torch.bfloat16, device=self.device)
        ops.relay_final(pend[0], pend[2], resid, pend[1], eps, out.view(-1), rs.epoch, rs.status)
        return out

    def _relay_decode_ok(self, B: int, key_bias, n_keys_max: int) -> bool:
        """Whether the relay covers this step: one row, the chained block's conditions, every launch shape covered
        (decided once per model) and an attention launch whose chunks merge inside the kernel."""
        if not RELAY or B != 1:
            return False
        if self._relay is None:
            if torch.cuda.is_current_stream_capturing():
                return False  # not decided yet: its buffers are not made inside a capture
            self._relay = _RelayState(self)
        rs = self._relay
        if n_keys_max not in rs.attn_ok:
            if torch.cuda.is_current_stream_capturing():
                return False
            c = self.config
            rs.attn_ok[n_keys_max] = ops.relay_footprint_attn(c.n_heads, c.head_dim, n_keys_max) is not None
            rs.plan(self, n_keys_max)
        return rs.covered and rs.attn_ok[n_keys_max]

    def relay_check(self) -> None:
        """Raises if a launch of the decode relay gave up waiting for its input since the last call (a host
        synchronisation; the results of that step are undefined)."""
        if self._relay is not None and int(self._relay.status[0].item()) != 0:
            words = self._relay.status.tolist()
            self._relay.status.zero_()
            raise RuntimeError(f"a launch of the decode relay gave up waiting for its producer (status words {words})")

    def _chain_decode_ok(self, M: int) -> bool:
        """Whether :meth:`_block_decode_chain` covers this model at ``M`` rows: decided once per ``M`` by
        issuing block 0's four linears in chained form on scratch inputs (outside any graph capture)."""
        cached = self._chain_ok.get(M)
        if cached is not None:
            return cached
        blk = self.transformer["blocks"][0]
        lin = (blk.att_proj, blk.attn_out, blk.ff_proj, blk.ff_out)
        ok = M <= 8 and all(isinstance(m, QuantLinear) for m in lin) and not torch.cuda.is_current_stream_capturing()
        if ok:
            d = self.config.d_model
            x = torch.zeros(M, 1, d, dtype=torch.bfloat16, device=self.device)
            nw = blk.attn_norm.weight.data
            s_in = torch.zeros(M, d // 16, dtype=torch.float32, device=self.device)
            r1 = ops.w4_linear_chain(x, blk.att_proj.tiled, resid=x, norm_w=nw, eps=1e-6, ssq_in=s_in, want_ssq=True)
            r2 = ops.w4_linear_chain(x, blk.attn_out.tiled, want_ssq=True)
            r3 = ops.w4_linear_chain(x, blk.ff_proj.tiled, resid=x, norm_w=nw, eps=1e-6, ssq_in=s_in, swiglu_out=True)
            ok = r1 is not None and r2 is not None and r3 is not None
            if ok:
                ok = ops.w4_linear_chain(r3[0], blk.ff_out.tiled, want_ssq=True) is not None
        elif torch.cuda.is_current_stream_capturing():
            return False  # not decided yet: do not record a probe into the graph
        self._chain_ok[M] = ok
        return ok

    # ------------------------------------------------------------------------------------------
    # forward: olmo/model.py:1253-1465
    # ------------------------------------------------------------------------------------------
    @torch.no_grad()
    def forward(
        self,
        input_ids: Optional[torch.LongTensor],
        input_embeddings: Optional[torch.Tensor] = None,
        attention_mask: Optional[torch.Tensor] = None,
        attention_bias: Optional[torch.Tensor] = None,
        past_key_values: Optional[Sequence[Tuple[torch.Tensor, torch.Tensor]]] = None,
        use_cache: bool = False,
        last_logits_only: bool = False,
        output_hidden_states: Optional[bool] = None,
        doc_lens: Optional[torch.Tensor] = None,
        max_doc_lens: Optional[Sequence[int]] = None,
    ) -> OLMoOutput:
        c = self.config
        if doc_lens is not None or max_doc_lens is not None:
            raise NotImplementedError("intra-document masking is a training feature and is not implemented")
        if not self._prepared:
            self.post_init()
        if past_key_values:
            assert len(past_key_values) == c.n_layers
        if input_embeddings is None:
            B, T = input_ids.shape
            x = self.transformer["wte"](input_ids.to(self.device))
        else:
            B, T = input_embeddings.shape[:2]
            x = input_embeddings.to(self.device, self.dtype).contiguous()

        # ---- cache ---------------------------------------------------------------------------
        cache: Optional[KVCache] = None
        if past_key_values:
            first = past_key_values[0]
            if isinstance(first, LayerKV):
                cache = first.cache
                past_len = first[0].size(-2)
                if past_len != cache.length:
                    cache.set_length(past_len)  # caller truncated / rewound the views
            else:
                cache = self._ingest_reference_cache(past_key_values, T)
                past_len = cache.length
            if cache.B != B:
                raise ValueError("batch size differs from the cache's")
            if past_len + T > cache.capacity:
                raise ValueError(f"KV cache capacity {cache.capacity} exceeded ({past_len}+{T}); "
                                 "construct the model with a larger max_cache_len")
        else:
            past_len = 0
            if use_cache:
                cache = self.new_cache(B, max(self.max_cache_len, T))

        # ---- padding mask -> additive per-key bias (olmo/model.py:1337-1340) ---------------------
        key_bias = None
        if attention_mask is not None:
            am = attention_mask.to(self.device, torch.float32).view(B, -1)
            if am.shape[1] != past_len + T:
                raise ValueError(f"attention_mask covers {am.shape[1]} positions, expected {past_len + T}")
            key_bias = ((1.0 - am) * torch.finfo(torch.float32).min).contiguous()
        if attention_bias is not None:
            kb = self.key_bias_from_attention_bias(attention_bias, B, past_len, past_len + T)
            key_bias = kb if key_bias is None else (key_bias + kb).contiguous()

        logits, hidden = self._forward_tokens(x, cache, B, T, past_len, key_bias, None, last_logits_only,
                                              bool(output_hidden_states))
        if cache is not None:
            cache.set_length(past_len + T)
        kvs = cache.views() if (use_cache and cache is not None) else None
        return OLMoOutput(logits=logits, attn_key_values=kvs, hidden_states=hidden)

    def key_bias_from_attention_bias(self, attention_bias: torch.Tensor, B: int, q0: int, q1: int) -> torch.Tensor:
        """An explicit ``attention_bias`` (``olmo/model.py:1343-1376``: ``[1 or B, 1, L, L]``, additive, or bool /
        int8 with 0 = masked) as the per-key bias ``[B, q1]`` the attention kernels take, for the query rows
        ``q0 .. q1-1``.  The kernels mask causally themselves and add one number per key, so the bias must be
        causal (every key after the query masked) and, below the diagonal, the same for every query row of the
        call: causal + padding, per-key penalties, anything for a single query row.  Other biases (ALiBi-like
        ones over several rows) raise ``NotImplementedError``.  Values are rounded to the activation dtype as the
        reference does (``olmo/model.py:516-531``)."""
        ab = attention_bias
        if ab.dim() != 4 or ab.shape[1] != 1 or ab.shape[0] not in (1, B) or ab.shape[2] < q1 or ab.shape[3] < q1:
            raise ValueError(f"attention_bias of shape {tuple(ab.shape)} does not cover {q1} positions of batch {B}")
        ab = ab.to(self.device)
        if ab.dtype in (torch.int8, torch.bool):
            ab = ab.to(torch.float32)
            ab = ab.masked_fill(ab == 0.0, torch.finfo(torch.float32).min)
        rows = ab[:, 0, q0:q1, :q1].to(torch.float32)  # [b, T, q1]
        kb = rows[:, -1, :]                            # the last row sees every key of the call
        qpos = torch.arange(q0, q1, device=self.device).view(1, -1, 1)
        future = torch.arange(q1, device=self.device).view(1, 1, -1) > qpos
        masked = rows <= -1e30
        same = (rows == kb.unsqueeze(1)) | (masked & (kb.unsqueeze(1) <= -1e30))
        if not bool((torch.where(future, masked, same)).all()):
            raise NotImplementedError("attention_bias must be causal and the same for every query row below the "
                                      "diagonal (causal + per-key terms); general biases are not implemented")
        if self.dtype != torch.float32:
            kb = kb.to(self.dtype).to(torch.float32)  # -inf where the dtype cannot hold the value: still masked
        return kb.expand(B, q1).contiguous()

    def _forward_tokens(self, x, cache: Optional[KVCache], B: int, T: int, past_len: int, key_bias, graph_pos,
                        last_logits_only: bool, collect_hidden: bool = False):
        """Blocks, final norm and head on embedded tokens ``x [B,T,d]``.  With ``graph_pos`` (device
        int32 holding the number of cached positions) the launch arguments do not depend on the
        position, so the call can be captured once and replayed; it requires ``T == 1``."""
        n_keys_max = cache.capacity if graph_pos is not None else past_len + T
        self._rope_now = cache.rope_now if (cache is not None and graph_pos is not None) else None
        hidden: List[torch.Tensor] = []
        self._beam = cache if isinstance(cache, BeamKVCache) else None
        if self._beam is not None and T != 1:
            raise ValueError("a beam cache takes one token per row")
        decode = T == 1 and cache is not None and self._beam is None
        fused = decode and self._fused_decode_ok(B, collect_hidden)
        chain = decode and self._fused_decode_ok(B, collect_hidden, rows_in_lds=False) and self._chain_decode_ok(B)
        pend = None
        if chain and self._relay_decode_ok(B, key_bias, n_keys_max):
            x = self._relay_blocks(x, cache, past_len, key_bias, graph_pos, n_keys_max)
            blocks = ()
        else:
            blocks = self.transformer["blocks"]
        for i, blk in enumerate(blocks):
            if collect_hidden:
                hidden.append(x)
            if cache is not None:
                kc, vc = cache.k[i], cache.v[i]
            else:
                kc, vc = self._scratch_cache(B, T)
            if chain:
                x, pend = self._block_decode_chain(blk, x, pend, kc, vc, B, past_len, key_bias, graph_pos, n_keys_max)
            elif fused:
                x, pend = self._block_decode_fused(blk, x, pend, kc, vc, B, past_len, key_bias, graph_pos, n_keys_max)
            else:
                x = self._block(blk, x, kc, vc, B, T, past_len, key_bias, graph_pos, n_keys_max)
        done = False
        if pend is not None:  # the last block's update has no following linear to ride on
            ln_f = self.transformer["ln_f"]
            w2 = getattr(ln_f, "weight", None)
            if not collect_hidden and isinstance(ln_f, RMSLayerNorm) and w2 is not None and ln_f.eps == self.config.layer_norm_eps:
                y = ops.rmsnorm_pair(pend[0], pend[1], x, w2.data, ln_f.eps)  # with the final norm, in one launch
                if y is not None:
                    x, done = y, True
            if not done:
                x = ops.rmsnorm(pend[0], pend[1], self.config.layer_norm_eps, residual=x)
        if last_logits_only and T > 1:
            x = x[:, -1, :].unsqueeze(1).contiguous()
        if not done:
            x = self.transformer["ln_f"](x)
        if collect_hidden:
            hidden.append(x)
        logits = self._head(x)
        return logits, (tuple(hidden) if collect_hidden else None)

    def _head(self, x: torch.Tensor) -> torch.Tensor:
        """Output projection; with weight tying the embedding matrix (``olmo/model.py:1454-1457``)."""
        if not self.config.weight_tying:
            return self._linear(self.transformer["ff_out"], x)
        wte = self.transformer["wte"].weight.data
        if wte.dtype == torch.float32:
            return ops.f32_linear(x, wte)
        return ops.b16_linear(x, self._tied_head)

    # ------------------------------------------------------------------------------------------
    # greedy generation: olmo/model.py:1603-1728 with beam_size 1 and the deterministic sampler
    # (olmo/beam_search.py:102-113): next = argmax(log_softmax(logits)) = argmax(logits)
    # ------------------------------------------------------------------------------------------
    @torch.no_grad()
    def generate(self, input_ids: torch.LongTensor, attention_mask: Optional[torch.Tensor] = None,
                 attention_bias: Optional[torch.Tensor] = None, max_steps: int = 10, beam_size: int = 1, per_node_beam_size: Optional[int] = None,
                 sampler=None, min_steps: Optional[int] = None, final_sequence_scorer=None,
                 constraints: Optional[list] = None, use_graph: bool = True, stop_at_eos: bool = True,
                 seed: int = 0) -> OLMoGenerateOutput:
        """``OLMo.generate`` (``olmo/model.py:1603-1728``).

        Beam size 1 without constraints, ``min_steps`` or a scorer is the captured greedy loop
        (``DeterministicSampler``), or one draw per step on the device with the ``MultinomialSampler`` /
        ``TopKSampler`` / ``TopPSampler`` of ``olmo_amd.beam_search``.  As in the reference's search a sequence
        that has emitted the end token only repeats it at no cost and the result is as long as the longest
        sequence (the captured loop looks for "all ended" every 16 steps; ``stop_at_eos=False`` runs all
        ``max_steps`` and leaves the tokens as generated).  Anything else is ``olmo_amd.beam_search.BeamSearch``
        over a :class:`BeamKVCache`.  ``scores`` is the
        summed log-probability of the chosen tokens under the unfiltered distribution (passed through
        ``final_sequence_scorer`` in a beam search)."""
        if attention_bias is not None:  # olmo/model.py:1645-1657
            B, P = input_ids.shape
            assert attention_bias.dim() == 4 and tuple(attention_bias.shape[:2]) == (B, 1)
            assert P + max_steps <= attention_bias.shape[2] == attention_bias.shape[3]
        plain = beam_size == 1 and not constraints and not min_steps and final_sequence_scorer is None
        if not plain:
            return self._generate_beam(input_ids, attention_mask, max_steps, beam_size, per_node_beam_size, sampler,
                                       min_steps, final_sequence_scorer, constraints, use_graph, attention_bias)
        from .generate import greedy_generate

        sampling = None
        if sampler is not None and not getattr(sampler, "greedy", False):
            if hasattr(sampler, "check"):
                sampler.check(self.config.logits_size)
            sampling = dict(sampler.params(), seed=seed)
        toks, scores = greedy_generate(self, input_ids, attention_mask, max_steps, use_graph=use_graph,
                                       eos_token_id=self.config.eos_token_id if stop_at_eos else None,
                                       return_scores=True, sampling=sampling, stop_when_all_ended=stop_at_eos,
                                       attention_bias=attention_bias)
        return OLMoGenerateOutput(token_ids=toks.unsqueeze(1), scores=scores.unsqueeze(1))

    def _generate_beam(self, input_ids, attention_mask, max_steps, beam_size, per_node_beam_size, sampler, min_steps,
                       final_sequence_scorer, constraints, use_graph: bool = True,
                       attention_bias: Optional[torch.Tensor] = None) -> OLMoGenerateOutput:
        """The step function of ``olmo/model.py:1677-1714`` for ``BeamSearch``: prefill once with the batch, then
        one token per beam and step against a :class:`BeamKVCache`; log-softmax of the last position on the
        device.  The model's part of a step (embedding to log-probabilities) is captured into a HIP graph after
        two eager steps: tokens, position and the row table are read from fixed device buffers."""
        from .beam_search import BeamSearch

        search = BeamSearch(self.config.eos_token_id, max_steps=max_steps, beam_size=beam_size,
                            per_node_beam_size=per_node_beam_size, sampler=sampler, min_steps=min_steps,
                            final_sequence_scorer=final_sequence_scorer, constraints=constraints)
        input_ids = input_ids.to(self.device)
        B, P = input_ids.shape
        if attention_mask is not None:
            assert attention_mask.shape == (B, P)
        if P + max_steps - 1 > self.max_cache_len:
            raise ValueError(f"prompt {P} + {max_steps} new tokens exceeds max_cache_len {self.max_cache_len}")
        model, c = self, self.config
        ab_keys = None  # attention_bias as a per-key bias over prompt + generated tokens
        if attention_bias is not None:
            ab_keys = self.key_bias_from_attention_bias(attention_bias, B, 0, P + max_steps - 1)

        class _Beams:  # the search's state: BeamSearch calls expand_beams once, reorder_beams after every step
            cache = None
            key_bias = None
            ids = None     # [rows, 1] tokens the step reads
            graph = None
            logp = None
            eager_steps = 0

            def expand_beams(st, batch: int, beam: int) -> None:
                pre = st.cache
                bc = BeamKVCache(c.n_layers, batch, beam, c.effective_n_kv_heads, P, max_steps, c.head_dim,
                                 model.dtype, model.device)
                for i in range(c.n_layers):  # the prompt, once per sequence
                    bc.k[i].view(batch, beam, *bc.k[i].shape[1:])[:, 0, :, :P] = pre.k[i][:, :, :P]
                    bc.v[i].view(batch, beam, *bc.v[i].shape[1:])[:, 0, :, :P] = pre.v[i][:, :, :P]
                bc.set_length(P)
                if attention_mask is not None or ab_keys is not None:
                    kb = torch.zeros(batch, beam, bc.capacity, dtype=torch.float32, device=model.device)
                    if attention_mask is not None:
                        am = attention_mask.to(model.device, torch.float32).view(batch, P)
                        kb[:, :, :P] = ((1.0 - am) * torch.finfo(torch.float32).min).unsqueeze(1)
                    if ab_keys is not None:
                        kb[:, :, : ab_keys.shape[1]] += ab_keys.unsqueeze(1)
                    st.key_bias = kb.view(batch * beam, bc.capacity)
                st.cache = bc

            def reorder_beams(st, backpointer: torch.Tensor) -> None:
                st.cache.reorder_beams(backpointer)

        def step(last_predictions: torch.Tensor, state: dict, timestep: int):
            st = state["beams"]
            if timestep == 0:
                out = model(input_ids, attention_mask=attention_mask, attention_bias=attention_bias, use_cache=True,
                            last_logits_only=True)
                st.cache = out.attn_key_values[0].cache
                logits = out.logits[:, -1]
            else:
                bc, R = st.cache, last_predictions.numel()
                if st.ids is None:
                    st.ids = torch.empty(R, 1, dtype=torch.int64, device=model.device)
                st.ids.copy_(last_predictions.view(R, 1))

                def run():
                    x = model.transformer["wte"](st.ids)
                    lg, _ = model._forward_tokens(x, bc, R, 1, 0, st.key_bias, bc.length_dev, True)
                    return ops.log_softmax(lg.reshape(R, -1))

                if st.graph is None and use_graph and st.eager_steps >= 2:
                    st.graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(st.graph):
                        st.logp = run()
                if st.graph is not None:
                    st.graph.replay()
                else:
                    st.logp = run()
                    st.eager_steps += 1
                bc.set_length(bc.length + 1)
                return st.logp, state
            return ops.log_softmax(logits.reshape(logits.shape[0], -1)), state

        tokens, scores = search.search(input_ids.new_zeros((B,)), {"beams": _Beams()}, step)
        return OLMoGenerateOutput(token_ids=tokens, scores=scores)

    @property
    def num_params(self) -> int:
        return sum(p.numel() for p in self.parameters())
