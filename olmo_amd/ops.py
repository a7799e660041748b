"""Torch-tensor front end of the C-ABI: shape / dtype / contiguity checks on the host, then a
call into ``libolmo355.so`` on the current torch stream.  PyTorch only provides device
memory and streams here; every computation is a HIP kernel of this package.

All functions require CUDA (ROCm) tensors and raise instead of falling back.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from ._lib import check, lib

F32, BF16, F16 = 0, 1, 2
_DT = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}
GEMV_MAX_M = 64


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported activation dtype {t.dtype}; float32, bfloat16 or float16") from None


def _dev(*ts: Optional[torch.Tensor]) -> None:
    dev = None
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("olmo_amd ops run on the GPU only (tensor is on %s); there is no CPU path" % t.device)
        if not t.is_contiguous():
            raise ValueError("tensor must be contiguous")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise ValueError("tensors on different devices")


def _p(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """Handle of torch's current stream on the current device.  The raw getter is ten times cheaper than building
    a ``torch.cuda.Stream`` object (2.7 us, a quarter of a launch's host time), which matters where launches are
    not replayed from a graph: short prefills are bound by the host."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


# ---------------------------------------------------------------------------------------------
# int4 weights
# ---------------------------------------------------------------------------------------------
def w4_dequant_fp16(qweight, qzeros, scales, group_size: int, g_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp16 ``[K, N]`` table, bit-exact with the reference's torch dequantize."""
    _dev(qweight, qzeros, scales, g_idx)
    if qweight.dtype != torch.int32 or qzeros.dtype != torch.int32 or scales.dtype != torch.float16:
        raise TypeError("qweight/qzeros must be int32 and scales float16")
    K, N = qweight.shape[0] * 8, qweight.shape[1]
    if g_idx is not None:
        if g_idx.dtype != torch.int32 or g_idx.numel() != K:
            raise ValueError("g_idx must be int32 [K]")
        G = scales.shape[0]
    else:
        G = K // group_size
    if scales.shape != (G, N) or qzeros.shape != (G, N // 8):
        raise ValueError(f"scales {tuple(scales.shape)} / qzeros {tuple(qzeros.shape)} do not match K={K} N={N} G={G}")
    out = torch.empty(K, N, dtype=torch.float16, device=qweight.device)
    check("olmo355_w4_dequant_fp16",
          lib().olmo355_w4_dequant_fp16(_p(qweight), _p(qzeros), _p(scales), _p(g_idx), _p(out), K, N, group_size,
                                        _stream()))
    return out


@dataclass
class W4Tiled:
    """An int4 weight in the MFMA-fragment layout (see include/olmo355.h)."""

    wt: torch.Tensor  # int32 [N/16, K/128, 64, 4]
    st: torch.Tensor  # float16 [N/16, K/128, 16]
    zt: torch.Tensor  # uint8 [N/16, K/128, 8]
    K: int
    N: int

    @property
    def nbytes(self) -> int:
        return self.wt.numel() * 4 + self.st.numel() * 2 + self.zt.numel()


def w4_repack(qweight, qzeros, scales, group_size: int) -> W4Tiled:
    _dev(qweight, qzeros, scales)
    K, N = qweight.shape[0] * 8, qweight.shape[1]
    if group_size != 128 or K % 128 or N % 16:
        raise ValueError(f"tiled int4 layout needs group_size 128, K % 128 == 0, N % 16 == 0 (got g={group_size}, K={K}, N={N})")
    G = K // 128
    if scales.shape != (G, N) or qzeros.shape != (G, N // 8):
        raise ValueError("scales / qzeros shape mismatch")
    dev = qweight.device
    wt = torch.empty(N // 16, G, 64, 4, dtype=torch.int32, device=dev)
    st = torch.empty(N // 16, G, 16, dtype=torch.float16, device=dev)
    zt = torch.empty(N // 16, G, 8, dtype=torch.uint8, device=dev)
    check("olmo355_w4_repack",
          lib().olmo355_w4_repack(_p(qweight), _p(qzeros), _p(scales), _p(wt), _p(st), _p(zt), K, N, group_size,
                                  _stream()))
    return W4Tiled(wt, st, zt, K, N)


def w4t_dequant_fp16(w: W4Tiled) -> torch.Tensor:
    _dev(w.wt, w.st, w.zt)
    out = torch.empty(w.K, w.N, dtype=torch.float16, device=w.wt.device)
    check("olmo355_w4t_dequant_fp16",
          lib().olmo355_w4t_dequant_fp16(_p(w.wt), _p(w.st), _p(w.zt), _p(out), w.K, w.N, _stream()))
    return out


def w4_linear_f16(x: torch.Tensor, w: W4Tiled) -> torch.Tensor:
    """``x[..., K] @ W[K, N]`` for a tiled int4 weight in the reference QuantLinear's own arithmetic: fp16 activations,
    weights dequantised to fp16, fp16 out (fp32 accumulation)."""
    _dev(x, w.wt)
    if x.dtype != torch.float16:
        raise TypeError("float16 activations expected")
    if x.shape[-1] != w.K:
        raise ValueError(f"x last dim {x.shape[-1]} != K {w.K}")
    M = x.numel() // w.K
    y = torch.empty(*x.shape[:-1], w.N, dtype=torch.float16, device=x.device)
    if M == 0:
        return y
    st = 2
    if M <= 16:
        st = lib().olmo355_w4_gemv_f16(_p(x), _p(w.wt), _p(w.st), _p(w.zt), _p(y), M, w.N, w.K, _stream())
        if st != 2:
            check("olmo355_w4_gemv_f16", st)
    if st == 2:
        check("olmo355_w4_gemm_f16", lib().olmo355_w4_gemm_f16(_p(x), _p(w.wt), _p(w.st), _p(w.zt), _p(y), M, w.N, w.K, _stream()))
    return y


def w4_linear(x: torch.Tensor, w: W4Tiled) -> torch.Tensor:
    """``x[..., K] @ W[K, N]`` for a tiled int4 weight; bf16 in, bf16 out (fp16 in, fp16 out: :func:`w4_linear_f16`)."""
    _dev(x, w.wt)
    if x.dtype == torch.float16:
        return w4_linear_f16(x, w)
    if x.dtype != torch.bfloat16:
        raise TypeError("int4 linear takes bfloat16 or float16 activations")
    if x.shape[-1] != w.K:
        raise ValueError(f"x last dim {x.shape[-1]} != K {w.K}")
    M = x.numel() // w.K
    y = torch.empty(*x.shape[:-1], w.N, dtype=torch.bfloat16, device=x.device)
    if M == 0:
        return y
    splits = _splitk(M, w.N, w.K) if M > 32 else 1
    if splits > 1:  # fewer tiles than CUs: several workgroups per tile along K, fp32 partials, one more kernel
        part = torch.empty(splits, M, w.N, dtype=torch.float32, device=x.device)
        check("olmo355_w4_gemm_splitk",
              lib().olmo355_w4_gemm_splitk(_p(x), _p(w.wt), _p(w.st), _p(w.zt), _p(y), M, w.N, w.K, splits, _p(part),
                                           _stream()))
    elif M <= GEMV_MAX_M:
        check("olmo355_w4_gemv",
              lib().olmo355_w4_gemv(_p(x), _p(w.wt), _p(w.st), _p(w.zt), _p(y), M, w.N, w.K, _stream()))
    else:
        ev = _gemm_begin()
        sk = _streamk(M, w.N, w.K, x.device)
        st = 2
        if sk is not None:
            st = lib().olmo355_w4_gemm_streamk(_p(x), _p(w.wt), _p(w.st), _p(w.zt), _p(y), M, w.N, w.K, _p(sk[0]),
                                               sk[0].numel(), sk[1], _stream())
            if st != 2:
                check("olmo355_w4_gemm_streamk", st)
        if st == 2:
            check("olmo355_w4_gemm",
                  lib().olmo355_w4_gemm(_p(x), _p(w.wt), _p(w.st), _p(w.zt), _p(y), M, w.N, w.K, _stream()))
        _gemm_end(ev, w.N, w.K, M)
    return y


class gemm_events:
    """``with gemm_events() as rec:`` puts a pair of HIP events around every many-row (M > 64) int4 linear issued
    meanwhile, on the stream it is issued on; after a synchronisation ``rec.rows()`` gives ``(N, K, M, seconds)`` per
    launch.  For measuring the GEMMs inside a real prefill; off (no events, no cost) otherwise."""
    active: Optional["gemm_events"] = None

    def __init__(self):
        self.items = []

    def __enter__(self):
        gemm_events.active = self
        return self

    def __exit__(self, *exc):
        gemm_events.active = None

    def rows(self):
        return [(n, k, m, e0.elapsed_time(e1) * 1e-3) for n, k, m, e0, e1 in self.items]


def _gemm_begin():
    if gemm_events.active is None:
        return None
    e0 = torch.cuda.Event(enable_timing=True)
    e0.record()
    return e0


def _gemm_end(e0, N: int, K: int, M: int) -> None:
    if e0 is not None and gemm_events.active is not None:
        e1 = torch.cuda.Event(enable_timing=True)
        e1.record()
        gemm_events.active.items.append((N, K, M, e0, e1))


SPLITK = True  # tests switch it off to compare the two forms
STREAMK = True  # likewise


def _splitk(M: int, N: int, K: int) -> int:
    return int(lib().olmo355_gemm_splitk_plan(M, N, K)) if SPLITK else 1


_streamk_ws = {}  # (device, stream) -> [workspace, epoch of its last launch]


def _streamk(M: int, N: int, K: int, device: torch.device):
    """``(workspace, epoch)`` for a stream-K launch of this shape on the current stream, or None when the tiled
    launch is the better one.  One buffer per (device, stream), zeroed once and kept for the life of the process:
    launches that share it are ordered on their stream, and each gets an epoch of its own (a counter that skips 0),
    so flags left by an earlier launch, finished or not, never pass for this one's."""
    if not STREAMK or not lib().olmo355_gemm_streamk_plan(M, N, K):
        return None
    if torch.cuda.is_current_stream_capturing():
        return None  # a captured launch would replay its epoch, and the flags of the last replay would pass for news
    key = (device.index if device.index is not None else torch.cuda.current_device(), _stream())
    slot = _streamk_ws.get(key)
    if slot is None:
        slot = [torch.zeros(int(lib().olmo355_gemm_streamk_workspace_bytes()), dtype=torch.uint8, device=device), 0]
        _streamk_ws[key] = slot
    slot[1] = slot[1] % 0x7FFFFFFF + 1
    return slot[0], slot[1]


def streamk_check() -> None:
    """Raise if a stream-K launch issued through this module gave up waiting for a partial (its tile then holds NaN).
    Reads one word per workspace back to the host (a synchronisation): for the end of a generation or a test, not
    for the path between launches.  The word is cleared, so one failure is reported once."""
    for (dev, _), (ws, _) in _streamk_ws.items():
        word = ws.view(torch.int32)[STREAMK_STATUS_WORD]
        epoch = int(word.item())
        if epoch:
            word.zero_()
            raise RuntimeError(f"a stream-K GEMM on device {dev} gave up waiting for a partial (launch epoch {epoch}): "
                               "its output holds NaN")


STREAMK_STATUS_WORD = 513  # O355_STREAMK_STATUS_WORD of the C header


# ---------------------------------------------------------------------------------------------
# dense weights
# ---------------------------------------------------------------------------------------------
@dataclass
class B16Tiled:
    wt: torch.Tensor  # bf16 or fp16 [N/16, K/32, 64, 8]
    K: int
    N: int


def b16_repack(weight_nk: torch.Tensor) -> B16Tiled:
    _dev(weight_nk)
    if weight_nk.dtype not in (torch.bfloat16, torch.float16) or weight_nk.dim() != 2:
        raise TypeError("expects a bfloat16 or float16 [N, K] weight")
    N, K = weight_nk.shape
    if K % 64 or N % 16:
        raise ValueError(f"dense 16-bit path needs K % 64 == 0 and N % 16 == 0 (got N={N}, K={K})")
    wt = torch.empty(N // 16, K // 32, 64, 8, dtype=weight_nk.dtype, device=weight_nk.device)
    check("olmo355_b16_repack", lib().olmo355_b16_repack(_p(weight_nk), _p(wt), N, K, _stream()))
    return B16Tiled(wt, K, N)


def f16_linear(x: torch.Tensor, w: B16Tiled) -> torch.Tensor:
    """``x @ W.T`` for fp16 activations and fp16 weights (fp32 accumulate, one rounding to fp16)."""
    _dev(x, w.wt)
    if x.dtype != torch.float16 or w.wt.dtype != torch.float16:
        raise TypeError("dense fp16 linear takes float16 activations and weights")
    if x.shape[-1] != w.K:
        raise ValueError(f"x last dim {x.shape[-1]} != K {w.K}")
    M = x.numel() // w.K
    y = torch.empty(*x.shape[:-1], w.N, dtype=torch.float16, device=x.device)
    if M:
        check("olmo355_f16_gemm", lib().olmo355_f16_gemm(_p(x), _p(w.wt), _p(y), M, w.N, w.K, _stream()))
    return y


def b16_linear(x: torch.Tensor, w: B16Tiled) -> torch.Tensor:
    _dev(x, w.wt)
    if w.wt.dtype == torch.float16:
        return f16_linear(x, w)
    if x.dtype != torch.bfloat16:
        raise TypeError("dense bf16 linear takes bfloat16 activations")
    if x.shape[-1] != w.K:
        raise ValueError(f"x last dim {x.shape[-1]} != K {w.K}")
    M = x.numel() // w.K
    y = torch.empty(*x.shape[:-1], w.N, dtype=torch.bfloat16, device=x.device)
    if M == 0:
        return y
    if M <= GEMV_MAX_M:
        check("olmo355_b16_gemv", lib().olmo355_b16_gemv(_p(x), _p(w.wt), _p(y), M, w.N, w.K, _stream()))
    else:
        splits = _splitk(M, w.N, w.K)
        if splits > 1:
            part = torch.empty(splits, M, w.N, dtype=torch.float32, device=x.device)
            check("olmo355_b16_gemm_splitk",
                  lib().olmo355_b16_gemm_splitk(_p(x), _p(w.wt), _p(y), M, w.N, w.K, splits, _p(part), _stream()))
        else:
            sk = _streamk(M, w.N, w.K, x.device)
            st = 2
            if sk is not None:
                st = lib().olmo355_b16_gemm_streamk(_p(x), _p(w.wt), _p(y), M, w.N, w.K, _p(sk[0]), sk[0].numel(), sk[1],
                                                    _stream())
                if st != 2:
                    check("olmo355_b16_gemm_streamk", st)
            if st == 2:
                check("olmo355_b16_gemm", lib().olmo355_b16_gemm(_p(x), _p(w.wt), _p(y), M, w.N, w.K, _stream()))
    return y


def linear_fused(x: torch.Tensor, w, resid: Optional[torch.Tensor] = None, norm_w: Optional[torch.Tensor] = None,
                 eps: float = 0.0, swiglu_out: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """Decode-step linear with its neighbours folded into the same launch: returns ``(y, x_new)`` with
    ``x_new = resid + rmsnorm(x; norm_w, eps)`` (``x`` itself without ``resid``) and
    ``y = x_new @ W`` (``swiglu(x_new @ W)`` with ``swiglu_out``).  Falls back to the separate kernels
    for shapes the fused kernels do not cover.  ``w``: ``W4Tiled`` or ``B16Tiled``."""
    _dev(x, resid, norm_w)
    if x.dtype != torch.bfloat16:
        raise TypeError("bfloat16 activations expected")
    M = x.numel() // w.K
    n_out = w.N // 2 if swiglu_out else w.N
    if M and M <= 16 and (resid is not None or swiglu_out):
        y = torch.empty(*x.shape[:-1], n_out, dtype=torch.bfloat16, device=x.device)
        x_new = torch.empty_like(x) if resid is not None else x
        xo = _p(x_new) if resid is not None else None
        if isinstance(w, W4Tiled):
            st = lib().olmo355_w4_gemv_fused(_p(x), _p(resid), _p(norm_w), float(eps), xo, _p(w.wt), _p(w.st), _p(w.zt),
                                             _p(y), M, w.N, w.K, int(swiglu_out), _stream())
            name = "olmo355_w4_gemv_fused"
        else:
            st = lib().olmo355_b16_gemv_fused(_p(x), _p(resid), _p(norm_w), float(eps), xo, _p(w.wt), _p(y), M, w.N, w.K,
                                              int(swiglu_out), _stream())
            name = "olmo355_b16_gemv_fused"
        if st == 0:
            return y, x_new
        if st != 2:
            check(name, st)
    x_new = rmsnorm(x, norm_w, eps, residual=resid) if resid is not None else x
    if swiglu_out and isinstance(w, W4Tiled) and M > GEMV_MAX_M:  # many rows: SwiGLU in the GEMM's epilogue
        y = torch.empty(*x.shape[:-1], n_out, dtype=torch.bfloat16, device=x.device)
        ev = _gemm_begin()
        sk = _streamk(M, w.N, w.K, x.device)
        st = 2
        if sk is not None:
            st = lib().olmo355_w4_gemm_swiglu_streamk(_p(x_new), _p(w.wt), _p(w.st), _p(w.zt), _p(y), M, w.N, w.K,
                                                     _p(sk[0]), sk[0].numel(), sk[1], _stream())
            if st not in (0, 2):
                check("olmo355_w4_gemm_swiglu_streamk", st)
        if st == 2:
            st = lib().olmo355_w4_gemm_swiglu(_p(x_new), _p(w.wt), _p(w.st), _p(w.zt), _p(y), M, w.N, w.K, _stream())
        if st == 0:
            _gemm_end(ev, w.N, w.K, M)
            return y, x_new
        if st != 2:
            check("olmo355_w4_gemm_swiglu", st)
    y = w4_linear(x_new, w) if isinstance(w, W4Tiled) else b16_linear(x_new, w)
    return (swiglu(y) if swiglu_out else y), x_new


def w4_linear_chain(x: torch.Tensor, w: "W4Tiled", resid: Optional[torch.Tensor] = None,
                    norm_w: Optional[torch.Tensor] = None, eps: float = 0.0, ssq_in: Optional[torch.Tensor] = None,
                    swiglu_out: bool = False, want_ssq: bool = False, r8_form: Optional[Tuple[int, int]] = None):
    """Decode-step int4 linear (at most 8 rows) with the norms chained between launches.  Returns
    ``(y, x_new, ssq)`` or ``None`` when the kernel does not cover the shape.  ``ssq`` (float32
    ``[M, N/16]``, only with ``want_ssq``) holds the sum of squares of every 16-column tile of ``y``: hand
    it to the launch that normalises ``y`` (``ssq_in`` here, ``qk_ssq`` of :func:`attn_decode_fused`).
    With ``resid``: ``x_new = resid + rmsnorm(x; norm_w, eps)`` using ``ssq_in`` for the mean square.
    ``r8_form=(tiles per workgroup, waves)`` (0 = choose) sends the call through the variant entry of the kernel for
    5 to 8 rows, for tests and tuning."""
    _dev(x, resid, norm_w, ssq_in)
    if x.dtype != torch.bfloat16 or not isinstance(w, W4Tiled):
        return None
    M = x.numel() // w.K
    if M < 1 or M > 8 or (resid is None) != (ssq_in is None) or (want_ssq and swiglu_out):
        return None
    n_out = w.N // 2 if swiglu_out else w.N
    y = torch.empty(*x.shape[:-1], n_out, dtype=torch.bfloat16, device=x.device)
    x_new = torch.empty_like(x) if resid is not None else x
    ssq = torch.empty(M, w.N // 16, dtype=torch.float32, device=x.device) if want_ssq else None
    args = (_p(x), _p(resid), _p(norm_w), float(eps), _p(x_new) if resid is not None else None, _p(ssq_in), _p(w.wt),
            _p(w.st), _p(w.zt), _p(y), _p(ssq), M, w.N, w.K, int(swiglu_out))
    if r8_form is None:
        st = lib().olmo355_w4_gemv_chain(*args, _stream())
    else:
        st = lib().olmo355_w4_gemv_r8_form(*args, int(r8_form[0]), int(r8_form[1]), _stream())
    if st == 2:
        return None
    check("olmo355_w4_gemv_chain", st)
    return y, x_new, ssq


RELAY_SPIN_LIMIT = 1 << 16  # polls of a waiting wave before it gives up and sets the status word (a tenth of a second)


def _spins(spin_limit: Optional[int]) -> int:
    return int(RELAY_SPIN_LIMIT if spin_limit is None else spin_limit)


def relay_untag(t: torch.Tensor) -> torch.Tensor:
    """Tagged words (int32: bf16 bits << 16 | epoch) -> the bf16 numbers (a copy)."""
    return t.contiguous().view(torch.int16).view(*t.shape, 2)[..., 1].contiguous().view(torch.bfloat16)


def relay_tags(t: torch.Tensor) -> torch.Tensor:
    """The 16-bit tags of tagged words."""
    return t & 0xFFFF


def relay_tag(x: torch.Tensor, out: torch.Tensor, epoch: torch.Tensor, stream: Optional[int] = None) -> torch.Tensor:
    """bf16 numbers -> tagged words carrying the current epoch, into ``out`` (int32, same count)."""
    _dev(x, out, epoch)
    if x.dtype != torch.bfloat16 or out.dtype != torch.int32 or out.numel() != x.numel() or epoch.dtype != torch.int32:
        raise TypeError("relay_tag: bf16 in, int32 out of the same size, int32 epoch")
    check("olmo355_relay_tag", lib().olmo355_relay_tag(_p(x), _p(out), x.numel(), _p(epoch), _stream() if stream is None else stream))
    return out


def w4_relay(x: torch.Tensor, w: "W4Tiled", y: torch.Tensor, epoch: torch.Tensor, status: torch.Tensor, *,
             resid: Optional[torch.Tensor] = None, norm_w: Optional[torch.Tensor] = None, eps: float = 0.0,
             ssq_in: Optional[torch.Tensor] = None, x_out: Optional[torch.Tensor] = None,
             ssq_out: Optional[torch.Tensor] = None, swiglu: bool = False, cfg: int = 0,
             hint_in: Optional[torch.Tensor] = None, hint_out: Optional[torch.Tensor] = None,
             spin_limit: Optional[int] = None, stream: Optional[int] = None) -> bool:
    """One int4 linear of the decode relay at one row; every buffer is the caller's (nothing is allocated).
    ``x``: int32 tagged words or bf16; ``y``: int32 (tagged) or bf16, ``N`` (``N/2`` with ``swiglu``) numbers;
    ``ssq_in`` / ``ssq_out``: int32 tagged sums per 16-column tile; ``resid`` / ``x_out``: tagged rows; with ``resid`` the
    activations are ``resid + rmsnorm(x; norm_w, eps)`` and also go to ``x_out``.  Returns ``False`` when the kernel
    does not cover the shape (nothing launched)."""
    _dev(x, y, epoch, status, resid, norm_w, ssq_in, x_out, ssq_out, w.wt)
    if x.numel() != w.K or x.dtype not in (torch.int32, torch.bfloat16) or y.dtype not in (torch.int32, torch.bfloat16):
        raise ValueError("w4_relay: one row of K tagged words or bf16 numbers in; int32 or bf16 out")
    if y.numel() != (w.N // 2 if swiglu else w.N):
        raise ValueError("w4_relay: output size mismatch")
    for t, n, dt in ((resid, w.K, torch.int32), (x_out, w.K, torch.int32), (norm_w, w.K, torch.bfloat16),
                     (ssq_in, w.K // 16, torch.int32), (ssq_out, w.N // 16, torch.int32)):
        if t is not None and (t.numel() != n or t.dtype != dt):
            raise ValueError("w4_relay: a side buffer has the wrong size or dtype")
    if epoch.dtype != torch.int32 or status.dtype != torch.int32 or status.numel() < 8:
        raise TypeError("w4_relay: an int32 epoch word and 8 int32 status words")
    st = lib().olmo355_w4_relay(_p(x), int(x.dtype == torch.int32), _p(ssq_in), _p(resid), _p(norm_w), float(eps), _p(x_out),
                                _p(w.wt), _p(w.st), _p(w.zt), _p(y), int(y.dtype == torch.int32), _p(ssq_out), w.N, w.K,
                                int(swiglu), _p(epoch), _p(status), _p(hint_in), _p(hint_out), _spins(spin_limit), int(cfg),
                                _stream() if stream is None else stream)
    if st == 2:
        return False
    check("olmo355_w4_relay", st)
    return True


def relay_final(x: torch.Tensor, ssq_in: torch.Tensor, resid: torch.Tensor, norm_w: torch.Tensor, eps: float,
                out: torch.Tensor, epoch: torch.Tensor, status: torch.Tensor, spin_limit: Optional[int] = None) -> torch.Tensor:
    """``out = resid + rmsnorm(x; norm_w, eps)`` from tagged rows into a plain bf16 row (the relay's last update)."""
    _dev(x, ssq_in, resid, norm_w, out, epoch, status)
    K = x.numel()
    if (x.dtype != torch.int32 or resid.dtype != torch.int32 or resid.numel() != K or ssq_in.dtype != torch.int32
            or ssq_in.numel() != K // 16 or norm_w.dtype != torch.bfloat16 or norm_w.numel() != K
            or out.dtype != torch.bfloat16 or out.numel() != K):
        raise ValueError("relay_final: tagged rows, int32 tagged sums, bf16 weight and output of one width expected")
    check("olmo355_relay_final",
          lib().olmo355_relay_final(_p(x), _p(ssq_in), _p(resid), _p(norm_w), float(eps), _p(out), K, _p(epoch), _p(status),
                                    _spins(spin_limit), _stream()))
    return out


def attn_decode_relay(qkv, q_weight, k_weight, sin_tab, cos_tab, kcache, vcache, ws, out, H: int, Hkv: int, hd: int,
                      past_len: int, n_keys_max: int, eps: float, epoch: torch.Tensor, status: torch.Tensor,
                      key_bias: Optional[torch.Tensor] = None, past_len_dev: Optional[torch.Tensor] = None,
                      qk_ssq: Optional[torch.Tensor] = None, rope_now: Optional[torch.Tensor] = None,
                      hint_in: Optional[torch.Tensor] = None, hint_out: Optional[torch.Tensor] = None,
                      spin_limit: Optional[int] = None, stream: Optional[int] = None) -> bool:
    """:func:`attn_decode_fused` for one sequence as a leg of the relay: ``qkv`` tagged words, ``qk_ssq`` int32 tagged sums,
    ``out`` tagged words ``[H * hd]``.  Returns ``False`` when the relay form does not cover the shape."""
    _dev(qkv, q_weight, k_weight, sin_tab, cos_tab, kcache, vcache, ws, out, key_bias, past_len_dev, qk_ssq, rope_now, epoch, status)
    width = (H + 2 * Hkv) * hd
    if qkv.dtype != torch.int32 or qkv.numel() != width or out.dtype != torch.int32 or out.numel() != H * hd:
        raise ValueError("attn_decode_relay: tagged qkv of one token and a tagged output row expected")
    if qk_ssq is not None and (qk_ssq.dtype != torch.int32 or qk_ssq.numel() != width // 16):
        raise ValueError("attn_decode_relay: qk_ssq int32 [(H + 2 Hkv) hd / 16] expected")
    if kcache.dtype != torch.bfloat16 or kcache.shape != vcache.shape or kcache.shape[1] != Hkv or kcache.shape[3] != hd:
        raise ValueError("attn_decode_relay: bf16 caches [B, Hkv, Lmax, hd] expected")
    if rope_now is not None and (rope_now.dtype != torch.float32 or rope_now.numel() != 2 * hd):
        raise ValueError("rope_now: float32 [2 * hd] expected")
    Lmax, n_pos = kcache.shape[2], sin_tab.shape[0]
    if ws.numel() * ws.element_size() < int(lib().olmo355_attn_decode_workspace_bytes(1, H, hd, n_keys_max)):
        raise ValueError("attention workspace too small")
    st = lib().olmo355_attn_decode_relay(_p(qkv), _p(q_weight), _p(k_weight), _p(sin_tab), _p(cos_tab), _p(kcache), _p(vcache),
                                         _p(key_bias), _p(out), _p(ws), _nbytes(ws), 1, H, Hkv, hd, Lmax, n_pos, past_len,
                                         _p(past_len_dev),
                                         n_keys_max, key_bias.shape[1] if key_bias is not None else 0, float(eps), _p(qk_ssq),
                                         _p(rope_now), _p(epoch), _p(status), _p(hint_in), _p(hint_out), _spins(spin_limit),
                                         _stream() if stream is None else stream)
    if st == 2:
        return False
    check("olmo355_attn_decode_relay", st)
    return True


def relay_footprint_w4(N: int, K: int, norm: bool, swiglu: bool, cfg: int = 0, x_tagged: bool = True):
    """(workgroups, waves per workgroup, registers per lane, LDS bytes per workgroup) of a :func:`w4_relay` launch,
    or ``None`` when the kernel does not cover the shape."""
    import ctypes

    out = (ctypes.c_int * 4)()
    st = lib().olmo355_w4_relay_footprint(N, K, int(norm), int(x_tagged), int(swiglu), int(cfg), out)
    return tuple(out) if st == 0 else None


def relay_footprint_attn(H: int, hd: int, n_keys_max: int):
    import ctypes

    out = (ctypes.c_int * 4)()
    st = lib().olmo355_attn_decode_relay_footprint(1, H, hd, n_keys_max, out)
    return tuple(out) if st == 0 else None


def relay_device():
    """(CUs, bytes of LDS per CU) of the current device."""
    import ctypes

    out = (ctypes.c_int * 2)()
    check("olmo355_relay_device", lib().olmo355_relay_device(out))
    return int(out[0]), int(out[1])


def relay_pair_ok(older, younger, n_cu: int, lds_per_cu: int) -> bool:
    """Whether the younger launch, waiting on the older one's output, can never keep a workgroup of the older one
    from starting (footprints as above)."""
    import ctypes

    a, b = (ctypes.c_int * 4)(*older), (ctypes.c_int * 4)(*younger)
    return bool(lib().olmo355_relay_pair_ok(a, b, int(n_cu), int(lds_per_cu)))


def f32_linear(x: torch.Tensor, weight_nk: torch.Tensor) -> torch.Tensor:
    _dev(x, weight_nk)
    if x.dtype != torch.float32 or weight_nk.dtype != torch.float32:
        raise TypeError("expects float32")
    N, K = weight_nk.shape
    if x.shape[-1] != K:
        raise ValueError("shape mismatch")
    M = x.numel() // K
    y = torch.empty(*x.shape[:-1], N, dtype=torch.float32, device=x.device)
    if M:
        check("olmo355_f32_linear", lib().olmo355_f32_linear(_p(x), _p(weight_nk), _p(y), M, N, K, _stream()))
    return y


# ---------------------------------------------------------------------------------------------
# norms, activation, embedding
# ---------------------------------------------------------------------------------------------
def rmsnorm(x, weight: Optional[torch.Tensor], eps: float, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    _dev(x, weight, residual)
    d = x.shape[-1]
    if weight is not None and (weight.dtype != x.dtype or weight.numel() != d):
        raise ValueError("weight must match x's dtype and last dim")
    if residual is not None and (residual.dtype != x.dtype or residual.shape != x.shape):
        raise ValueError("residual must match x")
    out = torch.empty_like(x)
    rows = x.numel() // d
    if rows:
        check("olmo355_rmsnorm",
              lib().olmo355_rmsnorm(_p(x), _p(weight), _p(residual), _p(out), rows, d, float(eps), _dt(x), _stream()))
    return out


def rmsnorm_pair(x, w1: torch.Tensor, residual: torch.Tensor, w2: torch.Tensor, eps: float) -> Optional[torch.Tensor]:
    """``rmsnorm(residual + rmsnorm(x; w1); w2)`` in one launch, bit-identical to the two :func:`rmsnorm` calls
    (the end of a decode step: the last block's update, then the final norm); ``None`` for widths the kernel
    does not take."""
    _dev(x, w1, residual, w2)
    d = x.shape[-1]
    if any(w.dtype != x.dtype or w.numel() != d for w in (w1, w2)) or residual.dtype != x.dtype or residual.shape != x.shape:
        raise ValueError("weights and residual must match x")
    out = torch.empty_like(x)
    rows = x.numel() // d
    if not rows:
        return out
    st = lib().olmo355_rmsnorm_pair(_p(x), _p(w1), _p(residual), _p(w2), _p(out), rows, d, float(eps), _dt(x), _stream())
    if st == 2:
        return None
    check("olmo355_rmsnorm_pair", st)
    return out


def layernorm_np(x: torch.Tensor, eps: float) -> torch.Tensor:
    _dev(x)
    d = x.shape[-1]
    out = torch.empty_like(x)
    rows = x.numel() // d
    if rows:
        check("olmo355_layernorm_np", lib().olmo355_layernorm_np(_p(x), _p(out), rows, d, float(eps), _dt(x), _stream()))
    return out


def swiglu(x: torch.Tensor) -> torch.Tensor:
    _dev(x)
    h2 = x.shape[-1]
    if h2 % 2:
        raise ValueError("last dim must be even")
    h = h2 // 2
    out = torch.empty(*x.shape[:-1], h, dtype=x.dtype, device=x.device)
    rows = x.numel() // h2
    if rows:
        check("olmo355_swiglu", lib().olmo355_swiglu(_p(x), _p(out), rows, h, _dt(x), _stream()))
    return out


def clamp_(x: torch.Tensor, c: float) -> torch.Tensor:
    """In-place ``x.clamp_(-c, c)`` (``clip_qkv``)."""
    _dev(x)
    if x.numel():
        check("olmo355_clamp", lib().olmo355_clamp(_p(x), x.numel(), float(c), _dt(x), _stream()))
    return x


def gather_columns(x: torch.Tensor, perm: torch.Tensor) -> torch.Tensor:
    """``x[..., perm]`` for 16-bit activations (the column remap in front of an act-order int4 linear)."""
    _dev(x, perm)
    if x.element_size() != 2 or perm.dtype != torch.int32:
        raise TypeError("gather_columns takes 16-bit activations and an int32 permutation")
    K = x.shape[-1]
    if perm.numel() != K:
        raise ValueError(f"permutation of {perm.numel()} for {K} columns")
    out = torch.empty_like(x)
    M = x.numel() // K
    if M:
        check("olmo355_gather_columns", lib().olmo355_gather_columns(_p(x), _p(perm), _p(out), M, K, _stream()))
    return out


def embedding(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    _dev(ids, table)
    if ids.dtype != torch.int64:
        raise TypeError("ids must be int64")
    vocab, d = table.shape
    out = torch.empty(*ids.shape, d, dtype=table.dtype, device=table.device)
    if ids.numel():
        check("olmo355_embedding",
              lib().olmo355_embedding(_p(ids), _p(table), _p(out), ids.numel(), d, vocab, _dt(table), _stream()))
    return out


def add(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    _dev(a, b)
    if a.shape != b.shape or a.dtype != b.dtype:
        raise ValueError("shape/dtype mismatch")
    out = torch.empty_like(a)
    if a.numel():
        check("olmo355_add", lib().olmo355_add(_p(a), _p(b), _p(out), a.numel(), _dt(a), _stream()))
    return out


def add_bias(x: torch.Tensor, bias_f16: torch.Tensor) -> torch.Tensor:
    """``x + bias`` over the last axis: bf16 or fp16 rows, the fp16 bias buffer of a quantised Linear."""
    _dev(x, bias_f16)
    N = x.shape[-1]
    if x.dtype not in (torch.bfloat16, torch.float16) or bias_f16.dtype != torch.float16 or bias_f16.shape != (N,):
        raise ValueError("add_bias takes bf16 or fp16 rows and an fp16 bias of the row length")
    x = x.contiguous()
    out = torch.empty_like(x)
    if x.numel():
        fn = lib().olmo355_add_bias_bf16 if x.dtype == torch.bfloat16 else lib().olmo355_add_bias_f16
        check("olmo355_add_bias", fn(_p(x), _p(bias_f16.contiguous()), _p(out), x.numel() // N, N, _stream()))
    return out


def argmax(logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _dev(logits, out)
    n = logits.shape[-1]
    rows = logits.numel() // n
    if out is None:
        out = torch.empty(logits.shape[:-1], dtype=torch.int64, device=logits.device)
    check("olmo355_argmax", lib().olmo355_argmax(_p(logits), _p(out), rows, n, _dt(logits), _stream()))
    return out


def greedy_next(logits: torch.Tensor, ids_out: torch.Tensor, table: torch.Tensor, x_next: torch.Tensor,
                pos_dev: torch.Tensor, sin_tab: torch.Tensor, cos_tab: torch.Tensor, rope_now: torch.Tensor) -> None:
    """The end of a greedy decode step in one launch: :func:`argmax` of every row into ``ids_out`` (int64), the
    chosen tokens' embedding rows into ``x_next [rows, d]``, and :func:`rope_advance` by one position."""
    _dev(logits, ids_out, table, x_next, pos_dev, sin_tab, cos_tab, rope_now)
    n = logits.shape[-1]
    rows = logits.numel() // n
    d, hd = table.shape[1], sin_tab.shape[1]
    if ids_out.dtype != torch.int64 or ids_out.numel() != rows or x_next.numel() != rows * d:
        raise ValueError("ids_out int64 [rows] and x_next [rows, d] expected")
    if table.dtype != logits.dtype or x_next.dtype != logits.dtype or not table.is_contiguous() or not x_next.is_contiguous():
        raise TypeError("table and x_next: contiguous, of the logits' dtype")
    if pos_dev.dtype != torch.int32 or rope_now.dtype != torch.float32 or rope_now.numel() != 2 * hd:
        raise TypeError("pos_dev int32, rope_now float32 [2 * hd] expected")
    check("olmo355_greedy_next",
          lib().olmo355_greedy_next(_p(logits), _p(ids_out), _p(table), _p(x_next), rows, n, d, table.shape[0], _p(pos_dev),
                                    _p(sin_tab), _p(cos_tab), _p(rope_now), hd, sin_tab.shape[0], _dt(logits), _stream()))


def log_softmax(logits: torch.Tensor) -> torch.Tensor:
    """``F.log_softmax(logits, dim=-1)`` with float32 results (beam search's step normalisation)."""
    _dev(logits)
    logits = logits.contiguous()
    n = logits.shape[-1]
    out = torch.empty(logits.shape, dtype=torch.float32, device=logits.device)
    check("olmo355_log_softmax", lib().olmo355_log_softmax(_p(logits), _p(out), logits.numel() // n, n, _dt(logits), _stream()))
    return out


def topk(x: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """``torch.topk(x, k, dim=-1)`` of float32 rows, sorted; equal values come in ascending index order."""
    _dev(x)
    if x.dtype != torch.float32:
        raise TypeError("topk: float32 expected")
    x = x.contiguous()
    n = x.shape[-1]
    rows = x.numel() // n
    vals = torch.empty(*x.shape[:-1], k, dtype=torch.float32, device=x.device)
    idx = torch.empty(*x.shape[:-1], k, dtype=torch.int64, device=x.device)
    check("olmo355_topk", lib().olmo355_topk(_p(x), rows, n, int(k), _p(vals), _p(idx), _stream()))
    return vals, idx


def gumbel_perturb(x: torch.Tensor, inv_temp: float = 1.0, seed: int = 0, counter: int = 0) -> torch.Tensor:
    """``x * inv_temp`` plus Gumbel(0, 1) noise per element (float32 rows); ``topk`` of the result draws without
    replacement from ``softmax(x * inv_temp)``."""
    _dev(x)
    if x.dtype != torch.float32:
        raise TypeError("gumbel_perturb: float32 expected")
    x = x.contiguous()
    n = x.shape[-1]
    out = torch.empty_like(x)
    check("olmo355_gumbel_perturb",
          lib().olmo355_gumbel_perturb(_p(x), _p(out), x.numel() // n, n, float(inv_temp), int(seed) & (2**64 - 1),
                                       int(counter) & (2**64 - 1), _stream()))
    return out


def gumbel_with_max(phi: torch.Tensor, row_max: torch.Tensor, seed: int = 0, counter: int = 0) -> torch.Tensor:
    """Gumbel(``phi``) samples per row ``[rows, n]`` conditioned on their maximum being ``row_max[row]``
    (``GumbelSampler.gumbel_with_max``)."""
    _dev(phi, row_max)
    if phi.dtype != torch.float32 or row_max.dtype != torch.float32:
        raise TypeError("gumbel_with_max: float32 expected")
    phi = phi.contiguous()
    n = phi.shape[-1]
    rows = phi.numel() // n
    if row_max.numel() != rows:
        raise ValueError("one maximum per row expected")
    out = torch.empty_like(phi)
    check("olmo355_gumbel_with_max",
          lib().olmo355_gumbel_with_max(_p(phi), _p(row_max.contiguous()), _p(out), rows, n, int(seed) & (2**64 - 1),
                                        int(counter) & (2**64 - 1), _stream()))
    return out


def sample(logits: torch.Tensor, temperature: float = 1.0, top_k: int = 0, top_p: float = 1.0, seed: int = 0,
           counter: int = 0, counter_dev: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
           logprob: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """One sampled token per row of ``logits``: temperature, then top-k, then top-p, then the draw.  Returns
    ``(tokens int64, log-probabilities float32)``; the log-probability is the chosen token's under the unscaled,
    unfiltered distribution.  The random number is a function of ``(seed, counter, row)``; ``counter_dev``
    (a device int32) overrides ``counter``."""
    _dev(logits, counter_dev, out, logprob)
    if not temperature > 0:
        raise ValueError("temperature must be positive")
    if top_k < 0 or not 0.0 <= top_p <= 1.0:
        raise ValueError("top_k must be >= 0 and top_p in [0, 1]")
    n = logits.shape[-1]
    rows = logits.numel() // n
    if out is None:
        out = torch.empty(logits.shape[:-1], dtype=torch.int64, device=logits.device)
    if logprob is None:
        logprob = torch.empty(logits.shape[:-1], dtype=torch.float32, device=logits.device)
    if counter_dev is not None and counter_dev.dtype != torch.int32:
        raise TypeError("counter_dev must be int32")
    check("olmo355_sample",
          lib().olmo355_sample(_p(logits), rows, n, float(temperature), int(top_k), float(top_p),
                               int(seed) & 0xFFFFFFFFFFFFFFFF, _p(counter_dev), int(counter), _p(out), _p(logprob),
                               _dt(logits), _stream()))
    return out, logprob


def incr_i32(p: torch.Tensor) -> None:
    _dev(p)
    if p.dtype != torch.int32:
        raise TypeError("int32 expected")
    check("olmo355_incr_i32", lib().olmo355_incr_i32(_p(p), _stream()))


# ---------------------------------------------------------------------------------------------
# attention
# ---------------------------------------------------------------------------------------------
def qknorm_rope_kvwrite(qkv, q_weight, k_weight, sin_tab, cos_tab, kcache, vcache, B: int, T: int, H: int, Hkv: int,
                        hd: int, past_len: int, eps: float, past_len_dev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Returns q (normed + rotated) ``[B, T, H*hd]``; writes rotated k and v into the caches."""
    _dev(qkv, q_weight, k_weight, sin_tab, cos_tab, kcache, vcache, past_len_dev)
    if qkv.shape[-1] != (H + 2 * Hkv) * hd or qkv.numel() != B * T * (H + 2 * Hkv) * hd:
        raise ValueError("qkv shape mismatch")
    if kcache.shape != vcache.shape or kcache.dim() != 4 or kcache.shape[0] < B or kcache.shape[1] != Hkv or kcache.shape[3] != hd:
        raise ValueError(f"cache shape {tuple(kcache.shape)} does not fit B={B} Hkv={Hkv} hd={hd}")
    if kcache.dtype != qkv.dtype or sin_tab.dtype != torch.float32 or cos_tab.dtype != torch.float32:
        raise TypeError("cache dtype must equal activation dtype; sin/cos tables float32")
    if sin_tab.shape != cos_tab.shape or sin_tab.shape[-1] != hd:
        raise ValueError("sin/cos tables must be [n_pos, hd]")
    Lmax, n_pos = kcache.shape[2], sin_tab.shape[0]
    if past_len_dev is None and past_len + T > min(Lmax, n_pos):
        raise ValueError(f"past_len + T = {past_len + T} exceeds cache length {Lmax} or rotary table {n_pos}")
    q = torch.empty(B, T, H * hd, dtype=qkv.dtype, device=qkv.device)
    check("olmo355_qknorm_rope_kvwrite",
          lib().olmo355_qknorm_rope_kvwrite(_p(qkv), _p(q_weight), _p(k_weight), _p(sin_tab), _p(cos_tab), _p(q),
                                            _p(kcache), _p(vcache), B, T, H, Hkv, hd, Lmax, n_pos, past_len,
                                            _p(past_len_dev), float(eps), _dt(qkv), _stream()))
    return q


PREFILL_SPLIT = True  # tests switch it off to compare the two forms
_prefill_ws = {}  # (device, stream) -> zeroed workspace of the key-split prefill attention, grown on demand


def attn_prefill(q, kcache, vcache, B: int, T: int, H: int, Hkv: int, hd: int, past_len: int,
                 key_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention of ``T`` new tokens per sequence over the cache rows ``0 .. past_len + T - 1``.  Where the
    library says the key-split form pays (a launch of one or two rounds of very unequal workgroups) it gets a
    workspace, one per device and stream, kept for the life of the process (launches on a stream are ordered and
    each leaves its counters at zero)."""
    _dev(q, kcache, vcache, key_bias)
    Lmax = kcache.shape[2]
    if q.numel() != B * T * H * hd or kcache.dtype != q.dtype:
        raise ValueError("q shape / cache dtype mismatch")
    if key_bias is not None and (key_bias.dtype != torch.float32 or key_bias.dim() != 2 or key_bias.shape[0] < B):
        raise ValueError("key_bias must be float32 [B, n]")
    out = torch.empty(B, T, H * hd, dtype=q.dtype, device=q.device)
    stride = key_bias.shape[1] if key_bias is not None else 0
    need = int(lib().olmo355_attn_prefill_workspace_bytes(B, T, H, hd, past_len, _dt(q))) if PREFILL_SPLIT else 0
    if need and not torch.cuda.is_current_stream_capturing():
        key = (q.device.index if q.device.index is not None else torch.cuda.current_device(), _stream())
        ws = _prefill_ws.get(key)
        if ws is None or ws.numel() < need:
            ws = torch.zeros(need, dtype=torch.uint8, device=q.device)
            _prefill_ws[key] = ws
        check("olmo355_attn_prefill_ws",
              lib().olmo355_attn_prefill_ws(_p(q), _p(kcache), _p(vcache), _p(key_bias), _p(out), _p(ws), ws.numel(), B, T, H, Hkv,
                                            hd, Lmax, past_len, stride, _dt(q), _stream()))
        return out
    check("olmo355_attn_prefill",
          lib().olmo355_attn_prefill(_p(q), _p(kcache), _p(vcache), _p(key_bias), _p(out), B, T, H, Hkv, hd, Lmax,
                                     past_len, stride, _dt(q), _stream()))
    return out


def _nbytes(t: torch.Tensor) -> int:
    return t.numel() * t.element_size()


def attn_decode_workspace(B: int, H: int, hd: int, n_keys_max: int, device) -> torch.Tensor:
    n = int(lib().olmo355_attn_decode_workspace_bytes(B, H, hd, n_keys_max))
    return torch.zeros(n // 4, dtype=torch.float32, device=device)  # the ticket counters at its start begin at zero


def attn_decode(q, kcache, vcache, ws, B: int, H: int, Hkv: int, hd: int, past_len: int, n_keys_max: int,
                key_bias: Optional[torch.Tensor] = None, past_len_dev: Optional[torch.Tensor] = None,
                beam_src: Optional[torch.Tensor] = None, prompt_len: int = 0, beam: int = 1) -> torch.Tensor:
    """``beam_src`` (int32 ``[B, steps]``) switches to the beam-search form: prompt rows from the first beam of
    each sequence, the row of generated token ``i`` from cache row ``beam_src[b, i]``."""
    _dev(q, kcache, vcache, ws, key_bias, past_len_dev, beam_src)
    Lmax = kcache.shape[2]
    if q.numel() != B * H * hd or kcache.dtype != q.dtype:
        raise ValueError("q shape / cache dtype mismatch")
    need = int(lib().olmo355_attn_decode_workspace_bytes(B, H, hd, n_keys_max))
    if ws.numel() * ws.element_size() < need:
        raise ValueError("attention workspace too small")
    out = torch.empty(B, 1, H * hd, dtype=q.dtype, device=q.device)
    if beam_src is not None:
        if beam_src.dtype != torch.int32 or beam_src.dim() != 2 or beam_src.shape[0] != B or not beam_src.is_contiguous():
            raise ValueError("beam_src: contiguous int32 [B, steps] expected")
        check("olmo355_attn_decode_beam",
              lib().olmo355_attn_decode_beam(_p(q), _p(kcache), _p(vcache), _p(key_bias), _p(out), _p(ws), _nbytes(ws), B, H, Hkv, hd,
                                             Lmax, past_len, _p(past_len_dev), n_keys_max,
                                             key_bias.shape[1] if key_bias is not None else 0, _p(beam_src),
                                             beam_src.shape[1], int(prompt_len), int(beam), _dt(q), _stream()))
        return out
    check("olmo355_attn_decode",
          lib().olmo355_attn_decode(_p(q), _p(kcache), _p(vcache), _p(key_bias), _p(out), _p(ws), _nbytes(ws), B, H, Hkv, hd, Lmax,
                                    past_len, _p(past_len_dev), n_keys_max,
                                    key_bias.shape[1] if key_bias is not None else 0, _dt(q), _stream()))
    return out


def attn_decode_fused(qkv, q_weight, k_weight, sin_tab, cos_tab, kcache, vcache, ws, B: int, H: int, Hkv: int, hd: int,
                      past_len: int, n_keys_max: int, eps: float, key_bias: Optional[torch.Tensor] = None,
                      past_len_dev: Optional[torch.Tensor] = None, qk_ssq: Optional[torch.Tensor] = None,
                      rope_now: Optional[torch.Tensor] = None, merge: int = -1) -> Optional[torch.Tensor]:
    """One new token per sequence: QK-norm, rotary, cache append and attention in one pass.  Returns
    ``None`` when the fused kernel does not cover the shape (use the separate calls then).  ``merge`` other than
    -1 names how a head's key chunks are merged (the variant entry point: 0 in the kernel, 2 separate kernel)."""
    _dev(qkv, q_weight, k_weight, sin_tab, cos_tab, kcache, vcache, ws, key_bias, past_len_dev, qk_ssq, rope_now)
    if rope_now is not None and (rope_now.dtype != torch.float32 or rope_now.numel() != 2 * hd):
        raise ValueError("rope_now: float32 [2 * hd] expected")
    if qkv.dtype != torch.bfloat16 or hd not in (64, 128):
        return None
    if qk_ssq is not None and (qk_ssq.dtype != torch.float32 or qk_ssq.numel() != B * (H + 2 * Hkv) * hd // 16):
        raise ValueError("qk_ssq: float32 [B, (H + 2 Hkv) hd / 16] expected")
    if qkv.numel() != B * (H + 2 * Hkv) * hd or kcache.shape != vcache.shape or kcache.shape[1] != Hkv or kcache.shape[3] != hd:
        raise ValueError("qkv / cache shape mismatch")
    Lmax, n_pos = kcache.shape[2], sin_tab.shape[0]
    need = int(lib().olmo355_attn_decode_workspace_bytes(B, H, hd, n_keys_max))
    if ws.numel() * ws.element_size() < need:
        raise ValueError("attention workspace too small")
    out = torch.empty(B, 1, H * hd, dtype=qkv.dtype, device=qkv.device)
    args = (_p(qkv), _p(q_weight), _p(k_weight), _p(sin_tab), _p(cos_tab), _p(kcache), _p(vcache), _p(key_bias), _p(out),
            _p(ws), _nbytes(ws), B, H, Hkv, hd, Lmax, n_pos, past_len, _p(past_len_dev), n_keys_max,
            key_bias.shape[1] if key_bias is not None else 0, float(eps), _p(qk_ssq), _p(rope_now), _dt(qkv))
    if merge == -1:
        st = lib().olmo355_attn_decode_fused(*args, _stream())
    else:
        st = lib().olmo355_attn_decode_fused_merge(*args, int(merge), _stream())
    if st == 2:
        return None
    check("olmo355_attn_decode_fused", st)
    return out


def rope_advance(pos_dev: torch.Tensor, delta: int, sin_tab: torch.Tensor, cos_tab: torch.Tensor,
                 rope_now: torch.Tensor) -> None:
    """``pos_dev += delta`` (device int32) and ``rope_now = [sin_tab[pos] | cos_tab[pos]]``: run between
    captured decode steps so that the attention kernel never looks the rotary rows up by position."""
    _dev(pos_dev, sin_tab, cos_tab, rope_now)
    hd = sin_tab.shape[1]
    if pos_dev.dtype != torch.int32 or rope_now.dtype != torch.float32 or rope_now.numel() != 2 * hd:
        raise TypeError("pos_dev int32, rope_now float32 [2 * hd] expected")
    check("olmo355_rope_advance",
          lib().olmo355_rope_advance(_p(pos_dev), int(delta), _p(sin_tab), _p(cos_tab), _p(rope_now), hd, sin_tab.shape[0],
                                     _stream()))


def rope_tables(head_dim: int, theta: float, n_pos: int, device) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp32 sin / cos tables ``[n_pos, hd]`` built with the reference's expression
    (``olmo/model.py:285-296``) on the host so that device sin/cos differences cannot enter."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float) / head_dim))
    seq = torch.arange(n_pos, dtype=torch.float)
    freqs = seq[:, None] * inv_freq[None, :]
    pos = torch.cat((freqs, freqs), dim=-1)
    return pos.sin().contiguous().to(device), pos.cos().contiguous().to(device)
