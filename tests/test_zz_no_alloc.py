"""The entry point that allocates nothing (``olmo355_attn_decode_static``: the chunk partials of the decode
attention live in a device array of the library) against the entry point it is a variant of
(``olmo355_attn_decode`` with a caller-provided workspace): same kernels, so bit-equal outputs; two calls in a
row, the second with a smaller input, so stale partials of the first call must not matter."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _case(L, dev, B, H, Hkv, hd, Lctx, seed, dtype=torch.bfloat16):
    from olmo_amd import ops

    g = torch.Generator().manual_seed(seed)
    Lmax = Lctx + 40
    q = torch.randn(B, H * hd, generator=g).to(dtype).to(dev)
    kc = torch.randn(B, Hkv, Lmax, hd, generator=g).to(dtype).to(dev)
    vc = torch.randn(B, Hkv, Lmax, hd, generator=g).to(dtype).to(dev)
    ws = ops.attn_decode_workspace(B, H, hd, Lmax, dev)
    pos = torch.tensor([Lctx - 1], dtype=torch.int32, device=dev)
    ref = torch.empty(B, H * hd, dtype=dtype, device=dev)
    out = torch.full_like(ref, float("nan"))
    s = torch.cuda.current_stream().cuda_stream
    dt = 1 if dtype == torch.bfloat16 else 0
    print("no_alloc case", B, H, Hkv, hd, Lctx, flush=True)
    assert L.olmo355_attn_decode(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), None, ref.data_ptr(), ws.data_ptr(),
                                 ws.numel() * ws.element_size(), B, H, Hkv, hd, Lmax, 0, pos.data_ptr(), Lmax, 0, dt, s) == 0
    free_before = torch.cuda.mem_get_info()[0]
    assert L.olmo355_attn_decode_static(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), None, out.data_ptr(), B, H, Hkv, hd, Lmax,
                                        0, pos.data_ptr(), Lmax, 0, dt, s) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, ref)
    return free_before


def test_static_scratch_entry_matches_workspace_entry():
    from olmo_amd import _lib

    assert torch.cuda.is_available()
    L = _lib.lib()
    dev = torch.device("cuda:0")
    assert L.olmo355_attn_decode_static_max_bytes() == 16 << 20
    _case(L, dev, 4, 32, 32, 128, 2048, seed=1)           # 4 x 32 heads x 17 chunks
    free_before = _case(L, dev, 2, 8, 2, 64, 300, seed=2)  # smaller, right after: stale partials around it
    _case(L, dev, 1, 4, 4, 32, 77, seed=3, dtype=torch.float32)
    # no device memory was taken by the calls (the array is part of the loaded library)
    assert torch.cuda.mem_get_info()[0] >= free_before - (1 << 20)
    # beyond the fixed maximum: refused before anything is launched
    q = torch.zeros(1, device=dev)
    st = L.olmo355_attn_decode_static(q.data_ptr(), q.data_ptr(), q.data_ptr(), None, q.data_ptr(), 64, 64, 64, 128, 1 << 20,
                                      0, None, 1 << 20, 0, 1, torch.cuda.current_stream().cuda_stream)
    assert st == 4 and b"scratch" in L.olmo355_status_string(4)
