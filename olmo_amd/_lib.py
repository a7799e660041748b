"""ctypes binding of ``libolmo355.so`` (the C-ABI declared in ``include/olmo355.h``).

The library is the product's only compute path: if it is missing or fails to load, every
op raises ``Olmo355Unavailable`` -- there is no PyTorch or CPU fallback.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_uint64, c_void_p
from typing import Optional

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libolmo355.so")

__all__ = ["lib", "LIB_PATH", "Olmo355Unavailable", "Olmo355Error", "check", "EXPORTS"]


class Olmo355Unavailable(RuntimeError):
    pass


class Olmo355Error(RuntimeError):
    def __init__(self, fn: str, status: int, text: str):
        super().__init__(f"{fn} failed with status {status}: {text}")
        self.status = status


P, I, L, F = c_void_p, c_int, c_int64, c_float


# name -> (restype, argtypes); must list every symbol include/olmo355.h declares
EXPORTS = {
    "olmo355_version": (I, []),
    "olmo355_status_string": (c_char_p, [I]),
    "olmo355_w4_dequant_fp16": (I, [P, P, P, P, P, I, I, I, P]),
    "olmo355_w4_repack": (I, [P, P, P, P, P, P, I, I, I, P]),
    "olmo355_w4t_dequant_fp16": (I, [P, P, P, P, I, I, P]),
    "olmo355_w4_gemv": (I, [P, P, P, P, P, I, I, I, P]),
    "olmo355_w4_gemv_fused": (I, [P, P, P, F, P, P, P, P, P, I, I, I, I, P]),
    "olmo355_w4_gemv_chain": (I, [P, P, P, F, P, P, P, P, P, P, P, I, I, I, I, P]),
    "olmo355_b16_gemv_fused": (I, [P, P, P, F, P, P, P, I, I, I, I, P]),
    "olmo355_w4_gemm": (I, [P, P, P, P, P, I, I, I, P]),
    "olmo355_w4_gemm_swiglu": (I, [P, P, P, P, P, I, I, I, P]),
    "olmo355_b16_repack": (I, [P, P, I, I, P]),
    "olmo355_b16_gemv": (I, [P, P, P, I, I, I, P]),
    "olmo355_b16_gemm": (I, [P, P, P, I, I, I, P]),
    "olmo355_f16_gemm": (I, [P, P, P, I, I, I, P]),
    "olmo355_f32_linear": (I, [P, P, P, I, I, I, P]),
    "olmo355_rmsnorm": (I, [P, P, P, P, I, I, F, I, P]),
    "olmo355_rmsnorm_pair": (I, [P, P, P, P, P, I, I, F, I, P]),
    "olmo355_layernorm_np": (I, [P, P, I, I, F, I, P]),
    "olmo355_qknorm_rope_kvwrite": (I, [P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, P, F, I, P]),
    "olmo355_attn_prefill": (I, [P, P, P, P, P, I, I, I, I, I, I, I, I, I, P]),
    "olmo355_attn_prefill_workspace_bytes": (L, [I, I, I, I, I, I]),
    "olmo355_attn_prefill_ws": (I, [P, P, P, P, P, P, L, I, I, I, I, I, I, I, I, I, P]),
    "olmo355_attn_decode_workspace_bytes": (L, [I, I, I, I]),
    "olmo355_attn_decode": (I, [P, P, P, P, P, P, L, I, I, I, I, I, I, P, I, I, I, P]),
    "olmo355_attn_decode_static_max_bytes": (L, []),
    "olmo355_attn_decode_static": (I, [P, P, P, P, P, I, I, I, I, I, I, P, I, I, I, P]),
    "olmo355_attn_decode_fused": (I, [P, P, P, P, P, P, P, P, P, P, L, I, I, I, I, I, I, I, P, I, I, F, P, P, I, P]),
    "olmo355_attn_decode_beam": (I, [P, P, P, P, P, P, L, I, I, I, I, I, I, P, I, I, P, I, I, I, I, P]),
    "olmo355_log_softmax": (I, [P, P, I, I, I, P]),
    "olmo355_topk": (I, [P, I, I, I, P, P, P]),
    "olmo355_gumbel_perturb": (I, [P, P, I, I, F, c_uint64, c_uint64, P]),
    "olmo355_gumbel_with_max": (I, [P, P, P, I, I, c_uint64, c_uint64, P]),
    "olmo355_gemm_splitk_plan": (I, [I, I, I]),
    "olmo355_w4_gemm_splitk": (I, [P, P, P, P, P, I, I, I, I, P, P]),
    "olmo355_b16_gemm_splitk": (I, [P, P, P, I, I, I, I, P, P]),
    "olmo355_w4_gemv_f16": (I, [P, P, P, P, P, I, I, I, P]),
    "olmo355_w4_gemm_f16": (I, [P, P, P, P, P, I, I, I, P]),
    "olmo355_gemm_streamk_workspace_bytes": (L, []),
    "olmo355_gemm_streamk_plan": (I, [I, I, I]),
    "olmo355_w4_gemm_streamk": (I, [P, P, P, P, P, I, I, I, P, L, I, P]),
    "olmo355_w4_gemm_swiglu_streamk": (I, [P, P, P, P, P, I, I, I, P, L, I, P]),
    "olmo355_b16_gemm_streamk": (I, [P, P, P, I, I, I, P, L, I, P]),
    "olmo355_rope_advance": (I, [P, I, P, P, P, I, I, P]),
    "olmo355_swiglu": (I, [P, P, I, I, I, P]),
    "olmo355_embedding": (I, [P, P, P, I, I, I, I, P]),
    "olmo355_gather_columns": (I, [P, P, P, I, I, P]),
    "olmo355_clamp": (I, [P, L, F, I, P]),
    "olmo355_sample": (I, [P, I, I, F, I, F, c_uint64, P, I, P, P, I, P]),
    "olmo355_add": (I, [P, P, P, L, I, P]),
    "olmo355_add_bias_bf16": (I, [P, P, P, I, I, P]),
    "olmo355_add_bias_f16": (I, [P, P, P, I, I, P]),
    "olmo355_argmax": (I, [P, P, I, I, I, P]),
    "olmo355_greedy_next": (I, [P, P, P, P, I, I, I, I, P, P, P, P, I, I, I, P]),
    "olmo355_incr_i32": (I, [P, P]),
}

# variant entry points of include/olmo355_debug.h (the dispatcher's choice as an explicit argument; tests and tuning)
VARIANT_EXPORTS = {
    "olmo355_w4_relay": (I, [P, I, P, P, P, F, P, P, P, P, P, I, P, I, I, I, P, P, P, P, I, I, P]),
    "olmo355_w4_relay_footprint": (I, [I, I, I, I, I, I, P]),
    "olmo355_relay_pair_ok": (I, [P, P, I, I]),
    "olmo355_relay_device": (I, [P]),
    "olmo355_relay_final": (I, [P, P, P, P, F, P, I, P, P, I, P]),
    "olmo355_relay_tag": (I, [P, P, I, P, P]),
    "olmo355_attn_decode_relay": (I, [P, P, P, P, P, P, P, P, P, P, L, I, I, I, I, I, I, I, P, I, I, F, P, P, P, P, P, P, I, P]),
    "olmo355_attn_decode_relay_footprint": (I, [I, I, I, I, P]),
    "olmo355_probe_stream_read": (I, [P, L, P, P]),
    "olmo355_probe_stream_read_many": (I, [P, P, I, P, P]),
    "olmo355_probe_mfma_bf16": (I, [I, P, P, P]),
    "olmo355_probe_fill_lds": (I, [ctypes.c_uint32, P, P]),
    "olmo355_w4_gemm_tile": (I, [P, P, P, P, P, I, I, I, I, P]),
    "olmo355_b16_gemm_tile": (I, [P, P, P, I, I, I, I, P]),
    "olmo355_w4_gemm_streamk_patience": (I, [P, P, P, P, P, I, I, I, P, L, I, I, I, P]),
    "olmo355_w4_gemv_form": (I, [P, P, P, P, P, I, I, I, I, P]),
    "olmo355_w4_gemv_r8_form": (I, [P, P, P, F, P, P, P, P, P, P, P, I, I, I, I, I, I, P]),
    "olmo355_attn_decode_fused_merge": (I, [P, P, P, P, P, P, P, P, P, P, L, I, I, I, I, I, I, I, P, I, I, F, P, P, I, I, P]),
}

_lib: Optional[ctypes.CDLL] = None


def lib() -> ctypes.CDLL:
    """Load the shared library once; fail loudly when it is not there."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise Olmo355Unavailable(
                f"{LIB_PATH} is missing: build it with `python -m olmo_amd.build` (hipcc, gfx950). "
                "There is no fallback path."
            )
        try:
            h = ctypes.CDLL(LIB_PATH)
        except OSError as e:  # pragma: no cover
            raise Olmo355Unavailable(f"cannot load {LIB_PATH}: {e}") from e
        for name, (res, args) in {**EXPORTS, **VARIANT_EXPORTS}.items():
            fn = getattr(h, name)
            fn.restype = res
            fn.argtypes = args
        _lib = h
    return _lib


def check(fn_name: str, status: int) -> None:
    if status != 0:
        raise Olmo355Error(fn_name, status, lib().olmo355_status_string(status).decode())
