"""TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's int4 group-wise format.

Nothing in the product (``olmo_amd/``) may import this module; it is the checker used by
``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg.

Restates, for ``bits=4`` only, the storage format, ``pack`` and the torch dequantize branch
of AutoGPTQ's ``QuantLinear`` as vendored inside the reference
(``inference/compression/dependencies/AutoGPTQ/auto_gptq/nn_modules/qlinear/qlinear_cuda_old.py``,
abbreviated ``AGQ:qlinear_cuda_old.py`` below).

Pinned by (see tests/test_oracle_w4.py): the three known-answer vectors the reference's
own kernel tests hold (``AGQ/tests/test_q4.py:21-1048,1213-1733``), a scalar brute-force
loop over nibbles on tiny shapes, the pack->unpack round trip, and exactness properties
of the fp16 product (subnormal scales, zero scales).
"""

from __future__ import annotations

from typing import Optional

import numpy as np
import torch

__all__ = [
    "unpack_qweight",
    "unpack_qzeros",
    "dequantize",
    "dequantize_bruteforce",
    "pack_nibbles",
    "pack_linear",
    "linear_fp32",
    "random_quantized",
]


def unpack_qweight(qweight: torch.Tensor) -> torch.Tensor:
    """int32 ``[K/8, N]`` -> uint8-valued int32 ``[K, N]``; nibble ``j`` of row ``r`` is
    ``q[8r+j]`` (``AGQ:qlinear_cuda_old.py:122-130`` packs it; ``:256-260`` unpacks it)."""
    q = qweight.to(torch.int32)
    shifts = torch.arange(0, 32, 4, dtype=torch.int32).view(1, 8, 1)
    out = (q.unsqueeze(1) >> shifts) & 15  # arithmetic shift, then mask: same bits as logical
    return out.reshape(q.shape[0] * 8, q.shape[1])


def unpack_qzeros(qzeros: torch.Tensor) -> torch.Tensor:
    """int32 ``[G, N/8]`` -> int32 ``[G, N]`` holding the *effective* zero point
    ``stored + 1`` (``AGQ:qlinear_cuda_old.py:156-166`` stores ``zero-1``; ``:242-248`` adds 1)."""
    z = qzeros.to(torch.int32)
    shifts = torch.arange(0, 32, 4, dtype=torch.int32).view(1, 1, 8)
    out = ((z.unsqueeze(2) >> shifts) & 15) + 1
    return out.reshape(z.shape[0], z.shape[1] * 8)


def dequantize(qweight: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor, group_size: int,
               g_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The reference's torch dequantize (``AGQ:qlinear_cuda_old.py:241-285``):
    ``W[k,n] = fp16(scales[g,n] * int8(q[k,n] - zero[g,n]))`` with ``g = k // group_size``, or
    ``g = g_idx[k]`` when an act-order ``g_idx`` is given (the per-row gather of scale and zero,
    ``AGQ:qlinear_cuda.py:253-265``).

    The int8 difference lies in [-16, 14]; fp16 x int8 in torch promotes the int8 to fp16
    (exact) and multiplies in fp16, i.e. the exact product rounded once to nearest-even
    with subnormals kept.  Computed here as fp32 product (exact: 11-bit x 5-bit significands)
    followed by one fp32->fp16 rounding.  Returns fp16 ``[K, N]``.
    """
    q = unpack_qweight(qweight)  # [K,N]
    z = unpack_qzeros(qzeros)  # [G,N]
    K, N = q.shape
    g = torch.arange(K) // group_size if g_idx is None else g_idx.to(torch.int64)
    diff = (q - z[g]).to(torch.float32)
    w = scales.to(torch.float16).to(torch.float32)[g] * diff
    return w.to(torch.float16)


def dequantize_torch_literal(qweight, qzeros, scales, group_size):
    """Same op sequence as the reference lines (int8 tensors, fp16 multiply), kept as a
    cross-check of ``dequantize``: ``AGQ:qlinear_cuda_old.py:241-262,284-285``."""
    wf = torch.arange(0, 32, 4, dtype=torch.int32).unsqueeze(0)
    zeros = torch.bitwise_right_shift(torch.unsqueeze(qzeros, 2).expand(-1, -1, 8), wf.unsqueeze(0)).to(torch.int8)
    zeros = torch.bitwise_and(zeros, 15)
    zeros = zeros + 1
    zeros = zeros.reshape(-1, 1, zeros.shape[1] * zeros.shape[2])
    sc = scales.reshape(-1, 1, scales.shape[-1])
    weight = torch.bitwise_right_shift(torch.unsqueeze(qweight, 1).expand(-1, 8, -1), wf.unsqueeze(-1)).to(torch.int8)
    weight = torch.bitwise_and(weight, 15)
    weight = weight.reshape(-1, group_size, weight.shape[2])
    weight = sc * (weight - zeros)
    return weight.reshape(weight.shape[0] * weight.shape[1], weight.shape[2])


def dequantize_bruteforce(qweight, qzeros, scales, group_size) -> np.ndarray:
    """Scalar loop over every nibble (tiny shapes only). Uses Python ints for the bit work
    and numpy float16 for the single rounding."""
    qw = qweight.numpy().astype(np.int64) & 0xFFFFFFFF
    qz = qzeros.numpy().astype(np.int64) & 0xFFFFFFFF
    sc = scales.numpy().astype(np.float16)
    K, N = qw.shape[0] * 8, qw.shape[1]
    out = np.zeros((K, N), dtype=np.float16)
    for k in range(K):
        g = k // group_size
        for n in range(N):
            q = (int(qw[k >> 3, n]) >> (4 * (k & 7))) & 15
            z = ((int(qz[g, n >> 3]) >> (4 * (n & 7))) & 15) + 1
            out[k, n] = np.float16(np.float32(sc[g, n]) * np.float32(q - z))
    return out


def pack_nibbles(q: torch.Tensor, axis: int) -> torch.Tensor:
    """Pack values in [0,15] eight per int32 along ``axis`` (0: rows -> qweight layout,
    1: columns -> qzeros layout), little nibble first (``AGQ:qlinear_cuda_old.py:122-130,156-166``)."""
    a = q.numpy().astype(np.uint32)
    if axis == 0:
        a = a.reshape(a.shape[0] // 8, 8, a.shape[1])
        out = np.zeros((a.shape[0], a.shape[2]), dtype=np.uint32)
        for j in range(8):
            out |= a[:, j, :] << np.uint32(4 * j)
    else:
        a = a.reshape(a.shape[0], a.shape[1] // 8, 8)
        out = np.zeros((a.shape[0], a.shape[1]), dtype=np.uint32)
        for j in range(8):
            out |= a[:, :, j] << np.uint32(4 * j)
    return torch.from_numpy(out.view(np.int32).copy())


def pack_linear(weight: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor, group_size: int):
    """``QuantLinear.pack`` for a dense ``weight [N,K]`` with per-(n, group) ``scales [N,G]``
    and integer ``zeros [N,G]`` in [1,16] (``AGQ:qlinear_cuda_old.py:98-166``):
    ``q = round((W + s*z)/s)``, stored zero is ``z-1``.  Returns (qweight, qzeros, scales_fp16)."""
    W = weight.to(torch.float32)
    s = scales.t().contiguous()  # [G,N]
    z = zeros.t().contiguous().to(torch.float32)
    sz = z * s
    s16 = s.clone().half()
    K = W.shape[1]
    g = torch.arange(K) // group_size
    intw = torch.round((W.t() + sz[g]) / s16[g]).to(torch.int32)  # [K,N]
    intw = intw.clamp_(0, 15)
    qweight = pack_nibbles(intw, 0)
    qzeros = pack_nibbles((z - 1).to(torch.int32), 1)
    return qweight, qzeros, s16


def linear_fp32(x: torch.Tensor, w_fp16: torch.Tensor) -> torch.Tensor:
    """``x @ W`` with both operands widened to fp32 (the value the reference's fp16 matmul
    ``AGQ:qlinear_cuda_old.py:287`` approximates)."""
    return x.to(torch.float32) @ w_fp16.to(torch.float32)


def random_quantized(K: int, N: int, group_size: int = 128, seed: int = 0):
    """Synthetic int4 weights: uniform nibbles in qweight and qzeros, fp16 scales
    ``|N(0, 0.01)|``, sequential groups."""
    gen = torch.Generator().manual_seed(seed)
    G = K // group_size
    qweight = torch.randint(-(2**31), 2**31, (K // 8, N), dtype=torch.int64, generator=gen).to(torch.int32)
    qzeros = torch.randint(-(2**31), 2**31, (G, N // 8), dtype=torch.int64, generator=gen).to(torch.int32)
    scales = (torch.randn(G, N, generator=gen) * 0.01).abs().to(torch.float16)
    return qweight, qzeros, scales
