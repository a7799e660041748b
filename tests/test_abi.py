"""CPU-side checks of the drop-in boundary: the shared library loads, exports every symbol the
header declares, and rejects bad arguments before touching the GPU."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_header_symbols_are_exported_and_bound():
    from olmo_amd import _lib

    hdr = open(os.path.join(ROOT, "include", "olmo355.h")).read()
    declared = set(re.findall(r"\b(olmo355_\w+)\s*\(", hdr))
    assert declared, "no declarations found"
    assert declared == set(_lib.EXPORTS), (declared ^ set(_lib.EXPORTS))
    h = _lib.lib()
    for name in declared:
        assert getattr(h, name) is not None
    assert h.olmo355_version() >= 1
    assert b"unsupported" in h.olmo355_status_string(2)


def test_variant_header_symbols_are_exported_and_bound():
    from olmo_amd import _lib

    hdr = open(os.path.join(ROOT, "include", "olmo355_debug.h")).read()
    declared = set(re.findall(r"\b(olmo355_\w+)\s*\(", hdr))
    assert declared == set(_lib.VARIANT_EXPORTS), (declared ^ set(_lib.VARIANT_EXPORTS))
    h = _lib.lib()
    for name in declared:
        assert getattr(h, name) is not None
    # the choice is an argument, not state: a bad value is refused before anything is launched
    assert h.olmo355_w4_gemv_form(None, None, None, None, None, 1, 16, 128, 9, None) == 1


def test_library_exports_no_state_setters():
    """The drop-in library promises no process-global state: nothing named *_set_* or *debug* is exported."""
    import subprocess

    from olmo_amd import _lib

    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True, check=True).stdout
    names = [ln.split()[-1] for ln in out.splitlines() if " T " in ln and "olmo355_" in ln]
    assert names and not [n for n in names if "_set_" in n or "debug" in n]
    assert set(names) == set(_lib.EXPORTS) | set(_lib.VARIANT_EXPORTS)


def test_argument_checks_return_status_without_launching():
    from olmo_amd import _lib

    h = _lib.lib()
    assert h.olmo355_w4_gemv(None, None, None, None, None, 1, 16, 128, None) == 1
    assert h.olmo355_w4_dequant_fp16(None, None, None, None, None, 8, 8, 8, None) == 1
    assert h.olmo355_rmsnorm(None, None, None, None, 1, 8, 1e-6, 1, None) == 1
    # workspace sizing is pure host arithmetic
    assert h.olmo355_attn_decode_workspace_bytes(1, 32, 128, 2048) == 32 * 16 * 130 * 8 + 32 * 8


def test_sized_workspaces_are_checked_before_any_device_call():
    """Every entry that writes into a caller's workspace takes its size and refuses one that is too small with
    O355_EINVAL before touching the device (so this runs without a GPU; the pointers are never dereferenced).  The
    same calls with the full size are the GPU tests' business."""
    import ctypes

    from olmo_amd import _lib

    h = _lib.lib()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    B, H, Hkv, hd, Lmax, keys = 2, 32, 32, 128, 4096, 2048
    need = h.olmo355_attn_decode_workspace_bytes(B, H, hd, keys)
    assert need > 0
    for short in (0, need - 1):
        assert h.olmo355_attn_decode(p, p, p, None, p, p, short, B, H, Hkv, hd, Lmax, 10, None, keys, 0, 0, None) == 1
        assert h.olmo355_attn_decode_beam(p, p, p, None, p, p, short, B, H, Hkv, hd, Lmax, 10, None, keys, 0, p, Lmax, 0, 2,
                                          0, None) == 1
        assert h.olmo355_attn_decode_fused(p, None, None, p, p, p, p, None, p, p, short, B, H, Hkv, hd, Lmax, Lmax, 10, None,
                                           keys, 0, 1e-6, None, None, 0, None) == 1
        assert h.olmo355_attn_decode_fused_merge(p, None, None, p, p, p, p, None, p, p, short, B, H, Hkv, hd, Lmax, Lmax, 10,
                                                 None, keys, 0, 1e-6, None, None, 0, 2, None) == 1
        assert h.olmo355_attn_decode_relay(p, None, None, p, p, p, p, None, p, p, short // B, 1, H, Hkv, hd, Lmax, Lmax, 10, None,
                                           keys, 0, 1e-6, None, None, p, p, None, None, 16, None) == 1
    # the key-split prefill attention: a workspace only where that form is taken; too small a one is refused
    pw = h.olmo355_attn_prefill_workspace_bytes
    assert pw(1, 2048, 16, 128, 0, 1) == 4096 + 16 * 8 * 2 * (4 * 2 * 8 * 64 * 16 + 4 * 2 * 64 * 8)
    assert pw(1, 2048, 32, 128, 0, 1) == 4096 + 32 * 4 * 2 * (4 * 2 * 8 * 64 * 16 + 4 * 2 * 64 * 8)  # every place taken: runs of 12
    assert pw(1, 1536, 40, 128, 0, 1) == 0 and pw(1, 1024, 16, 128, 0, 1) == 0 and pw(1, 2048, 16, 128, 5, 1) == 0
    assert pw(8, 2048, 32, 128, 0, 1) == 0  # several rounds of workgroups balance themselves
    assert pw(1, 2048, 16, 128, 0, 0) == 0 and pw(1, 2048, 16, 32, 0, 1) == 0 and pw(1, 8192, 2, 128, 0, 1) == 0
    assert h.olmo355_attn_prefill_ws(p, p, p, None, p, p, pw(1, 2048, 16, 128, 0, 1) - 1, 1, 2048, 16, 16, 128, 4096, 0, 0, 1,
                                     None) == 1
    need = h.olmo355_gemm_streamk_workspace_bytes()
    assert need == 4096 + 256 * 256 * 256 * 4
    for short, epoch in ((0, 1), (need - 1, 1), (need, 0)):  # epoch 0 is the value of a workspace never written: refused
        assert h.olmo355_w4_gemm_streamk(p, p, p, p, p, 2048, 12288, 4096, p, short, epoch, None) == 1
        assert h.olmo355_w4_gemm_swiglu_streamk(p, p, p, p, p, 2048, 22016, 4096, p, short, epoch, None) == 1
        assert h.olmo355_b16_gemm_streamk(p, p, p, 2048, 12288, 4096, p, short, epoch, None) == 1
        assert h.olmo355_w4_gemm_streamk_patience(p, p, p, p, p, 2048, 12288, 4096, p, short, epoch, 4, 0, None) == 1


def test_gemm_plans_are_host_arithmetic():
    """Which form a large-M product takes is decided on the host from the shape alone; the decisions that the 7B
    prefill rests on (measured: see the comments at the plan functions), kept from drifting."""
    from olmo_amd import _lib

    h = _lib.lib()
    sk, sp = h.olmo355_gemm_streamk_plan, h.olmo355_gemm_splitk_plan
    # one prompt of 2048 tokens: 384, 688 and 128 tiles of 256 x 256 -- stream-K where the rounds are uneven or K is long
    assert sk(2048, 12288, 4096) == 1 and sk(2048, 22016, 4096) == 1 and sk(2048, 4096, 11008) == 1
    assert sk(2048, 4096, 4096) == 0       # every tile would be shared and K is short: the tiled launch
    assert sk(8192, 4096, 4096) == 0       # 512 tiles: two full rounds
    assert sk(1024, 4096, 11008) == 1 and sk(1024, 4096, 4096) == 0   # 64 tiles: only a long K pays
    assert sk(512, 4096, 11008) == 0       # 32 tiles: split-K's range
    assert sk(2048, 4096, 4000) == 0       # K must divide into units of 256
    assert sp(512, 4096, 11008) == 2 and sp(300, 4096, 4096) == 2 and sp(2048, 4096, 4096) == 1
    assert sk(0, 4096, 4096) == 0 and sp(0, 4096, 4096) == 1


def test_ops_refuse_cpu_tensors():
    import torch

    from olmo_amd import ops

    with pytest.raises(RuntimeError, match="GPU only"):
        ops.rmsnorm(torch.zeros(2, 8), None, 1e-6)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from olmo_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.Olmo355Unavailable):
        _lib.lib()
