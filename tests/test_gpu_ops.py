"""GPU parity of every HIP kernel, called through the C-ABI, against the CPU oracle on the
same seeded inputs.  Integer / table work is bit-exact; floating point carries its tolerance
next to the assertion."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import model as om
from oracle import w4 as ow4

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from olmo_amd import _lib

    _lib.lib()  # fail loudly if the HIP library is not built
    return torch.device("cuda:0")


def _ops():
    from olmo_amd import ops

    return ops


def poison_lds(dev):
    """NaNs into the LDS of every CU: a kernel that reads LDS it has not written then shows it in its output
    (LDS keeps what the last workgroup left, often zeros, so such a read can pass unnoticed otherwise)."""
    from olmo_amd import _lib

    sink = torch.zeros(256, dtype=torch.int32, device=dev)
    assert _lib.lib().olmo355_probe_fill_lds(0x7FC07FC0, sink.data_ptr(), torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    assert int(sink.sum().item()) == 0


def say(*a):
    print(*a, flush=True)


# ------------------------------------------------------------------------------------------------
# int4 table: bit-exact
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("K,N,g", [(128, 16, 128), (256, 48, 128), (512, 64, 64), (4096, 256, 128), (1024, 1024, 128)])
def test_w4_dequant_bit_exact(dev, K, N, g):
    say("w4_dequant", K, N, g)
    ops = _ops()
    qw, qz, sc = ow4.random_quantized(K, N, g, seed=K * 7 + N)
    if K == 256:  # subnormal / zero / large scales must survive
        sc[0, :8] = torch.tensor([0.0, 6e-8, 1.2e-7, 3e-6, 5.9e-5, 6.2e-5, 1e-3, 4000.0], dtype=torch.float16)
    ref = ow4.dequantize(qw, qz, sc, g)
    out = ops.w4_dequant_fp16(qw.to(dev), qz.to(dev), sc.to(dev), g).cpu()
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))
    if g == 128 and N % 16 == 0:
        t = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), g)
        out2 = ops.w4t_dequant_fp16(t).cpu()
        assert torch.equal(out2.view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("N,K", [(4096, 4096), (11008, 4096), (4096, 11008), (13824, 5120), (100352, 4096)])
def test_w4_dequant_bit_exact_sweep_shapes(dev, N, K):
    """The shapes of the isolated linear sweep (`bench.py --sweep`): the fp16 table from the GPTQ tensors and
    from the tiled layout the timed kernels read, both bit-exact against the oracle."""
    say("w4_dequant sweep shape", N, K)
    ops = _ops()
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=N + K)
    # the oracle runs on column bands (all of them unless N is the vocabulary-sized one: first, middle, last)
    bands = [(0, N)] if N <= 20000 else [(0, 4096), (N // 2 - 2048, N // 2 + 2048), (N - 4096, N)]
    a = ops.w4_dequant_fp16(qw.to(dev), qz.to(dev), sc.to(dev), 128).view(torch.int16)
    b = ops.w4t_dequant_fp16(ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)).view(torch.int16)
    assert a.shape == b.shape == (K, N)
    for lo, hi in bands:
        ref = ow4.dequantize(qw[:, lo:hi].contiguous(), qz[:, lo // 8 : hi // 8].contiguous(), sc[:, lo:hi].contiguous(), 128)
        ref = ref.view(torch.int16)
        assert torch.equal(a[:, lo:hi].cpu(), ref), (lo, hi)
        assert torch.equal(b[:, lo:hi].cpu(), ref), (lo, hi)


def test_w4_dequant_g_idx_general(dev):
    ops = _ops()
    K, N, g = 256, 32, 128
    qw, qz, sc = ow4.random_quantized(K, N, g, seed=11)
    perm = torch.randperm(K, generator=torch.Generator().manual_seed(0))
    g_idx = (perm // g).to(torch.int32)
    q = ow4.unpack_qweight(qw)
    z = ow4.unpack_qzeros(qz)
    ref = (sc.float()[g_idx.long()] * (q - z[g_idx.long()]).float()).half()
    out = ops.w4_dequant_fp16(qw.to(dev), qz.to(dev), sc.to(dev), g, g_idx.to(dev)).cpu()
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


def _ulp16(ref):
    """One fp16 unit in the last place at the magnitude of ``ref`` (normal range)."""
    return torch.maximum(torch.tensor(2.0 ** -24), 2.0 ** (torch.floor(torch.log2(ref.abs().clamp_min(2.0 ** -14))) - 10))


def test_w4_golden_vectors_through_gemv(dev, golden_dir):
    """The reference's own kernel KATs (AGQ tests/test_q4.py:1071-1104, :1757-1764) through the HIP kernels in the
    reference's own arithmetic -- fp16 activations, fp16(scale * (q - zero)) weights: the decode kernel and, for the same
    single row, the tiled GEMM must both give the stored outputs to 2 fp16 ulp, with no allowance for input rounding.
    The bf16 path (the model's) is held to the oracle on the same bf16-rounded inputs."""
    import json
    import os

    from olmo_amd import _lib

    ops = _ops()
    kats = json.load(open(os.path.join(golden_dir, "q4_kat.json")))
    for name in ("exllama_k1024_n1024", "cuda_old_half_k256_n256", "cuda_old_no_half_k256_n256"):
        kat = kats[name]
        k, n = kat["k"], kat["n"]
        torch.manual_seed(42)
        qweight = torch.randint(-100, 100, size=(k // 8, n), dtype=torch.int32)
        scales = torch.zeros(k // 128, n, dtype=torch.float16) + 0.002
        qzeros = torch.zeros(k // 128, n // 8, dtype=torch.int32)
        inp = torch.rand(1, 1, k, dtype=torch.float16)
        t = ops.w4_repack(qweight.to(dev), qzeros.to(dev), scales.to(dev), 128)
        stored = torch.tensor(kat["out"])
        x16 = inp[0].to(dev)
        y16 = ops.w4_linear(x16, t)
        assert y16.dtype == torch.float16
        assert ((y16.float().cpu()[0] - stored).abs() <= 2 * _ulp16(stored)).all(), name
        yg = torch.empty_like(y16)
        assert _lib.lib().olmo355_w4_gemm_f16(x16.data_ptr(), t.wt.data_ptr(), t.st.data_ptr(), t.zt.data_ptr(), yg.data_ptr(), 1, n, k,
                                              torch.cuda.current_stream().cuda_stream) == 0
        assert ((yg.float().cpu()[0] - stored).abs() <= 2 * _ulp16(stored)).all(), name
        W = ow4.dequantize(qweight, qzeros, scales, 128)
        xb = inp[0].to(torch.bfloat16)
        y = ops.w4_linear(xb.to(dev), t).float().cpu()[0]
        assert torch.allclose(y, ow4.linear_fp32(xb, W)[0], rtol=2 ** -8, atol=1e-3), name


@pytest.mark.parametrize("M", [1, 3, 4, 5, 8, 9, 16, 17, 40, 300, 2048])
@pytest.mark.parametrize("N,K", [(4096, 4096), (1024, 11008), (272, 384)])
def test_w4_linear_fp16(dev, M, N, K):
    """fp16 activations (the reference QuantLinear's arithmetic) against the oracle on the same fp16 inputs and the
    fp16 dequantised table: one fp16 rounding of the result plus what fp32 sums of this length differ by."""
    say("w4_linear_fp16", M, N, K)
    ops = _ops()
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=M + N + K)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(7)).to(torch.float16)
    W = ow4.dequantize(qw, qz, sc, 128)
    ref = ow4.linear_fp32(x, W)
    t = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    y = ops.w4_linear(x.to(dev), t)
    assert y.dtype == torch.float16 and torch.equal(y, ops.w4_linear(x.to(dev), t))
    err = (y.float().cpu() - ref).abs()
    assert (err <= 2 * _ulp16(ref) + 2 ** -13 * ref.abs().max()).all(), float(err.max())


# ------------------------------------------------------------------------------------------------
# int4 linear: GEMV (M<=64) and GEMM paths
# ------------------------------------------------------------------------------------------------
def _w4_case(dev, M, N, K, seed):
    ops = _ops()
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=seed)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(seed + 1)).to(torch.bfloat16)
    W = ow4.dequantize(qw, qz, sc, 128)
    ref = ow4.linear_fp32(x, W)
    t = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    y = ops.w4_linear(x.to(dev), t)
    y2 = ops.w4_linear(x.to(dev), t)
    assert torch.equal(y, y2), "not deterministic"
    y = y.float().cpu()
    # bf16 output rounding (2^-9 relative) + fp32 accumulation noise; GEMM path also rounds W to bf16
    # (2^-9 relative per weight, averaging over K): budget 2^-7 relative to the row scale
    scale = ref.abs().max().item()
    err = (y - ref).abs().max().item()
    return err, scale


@pytest.mark.parametrize("M", [1, 2, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(256, 256), (4096, 4096), (1008, 1408)])
def test_w4_gemv(dev, M, N, K):
    say("w4_gemv", M, N, K)
    err, scale = _w4_case(dev, M, N, K, seed=M + N + K)
    assert err <= 2 ** -7 * scale, (err, scale)


@pytest.mark.parametrize("M", [5, 8, 9, 16, 17, 32, 48, 64])
@pytest.mark.parametrize("N,K", [(8208, 640), (11008, 4096), (4112, 128), (16, 1024), (16400, 256), (32784, 384)])
def test_w4_gemv_mid_rows(dev, M, N, K):
    """The kernel that stages the activations through LDS (every M > 16; from 9 rows at N >= 8192, from 8 at
    N >= 12288): one, two and four row tiles, both workgroup widths, an odd number of column tiles, and K
    that ends in the middle of a 512-wide stage or is shorter than one."""
    say("w4_gemv_mid", M, N, K)
    err, scale = _w4_case(dev, M, N, K, seed=M + N + K)
    assert err <= 2 ** -7 * scale, (err, scale)


@pytest.mark.parametrize("M,N,K", [(65, 256, 256), (128, 512, 1024), (300, 1008, 1408), (2048, 4096, 4096),
                                   (512, 12288, 4096)])
def test_w4_gemm(dev, M, N, K):
    say("w4_gemm", M, N, K)
    err, scale = _w4_case(dev, M, N, K, seed=M + N + K)
    assert err <= 2 ** -7 * scale, (err, scale)


def _w4_big_case(dev, N, K, Ms, seed):
    """The int4 linear at full layer sizes.  The oracle product is evaluated on column bands (all columns unless N is
    the vocabulary-sized one: first, middle and last 4096) and, above 64 rows, on a sample of rows (first and last
    tile rows and 24 random ones); at the largest M the whole output is additionally checked through a property
    that needs no oracle: permuting the rows of x permutes the rows of y -- bit for bit on the tiled launches; where
    the stream-K form runs, a row's fp32 partial sums are cut at a K that depends on its tile, so there the two agree
    to one rounding of the output and are bit-equal with stream-K switched off."""
    ops = _ops()
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=seed)
    t = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    bands = [(0, N)] if N <= 30000 else [(0, 4096), (N // 2 - 2048, N // 2 + 2048), (N - 4096, N)]
    Wb = [ow4.dequantize(qw[:, lo:hi].contiguous(), qz[:, lo // 8: hi // 8].contiguous(), sc[:, lo:hi].contiguous(), 128).float()
          for lo, hi in bands]
    for M in Ms:
        say("  M", M)
        g = torch.Generator().manual_seed(seed + M)
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        y = ops.w4_linear(x.to(dev), t)
        rows = torch.arange(M) if M <= 64 else torch.unique(torch.cat([
            torch.arange(0, 8), torch.arange(M - 8, M), torch.randint(0, M, (24,), generator=g)]))
        ysel = y[rows.to(dev)].float().cpu()
        for (lo, hi), W in zip(bands, Wb):
            ref = x[rows].float() @ W
            scale = ref.abs().max().item()
            err = (ysel[:, lo:hi] - ref).abs().max().item()
            assert err <= 2 ** -7 * scale, (M, lo, hi, err, scale)
        if M == max(Ms) and M > 64:
            perm = torch.randperm(M, generator=g)
            xp = x[perm].contiguous().to(dev)
            y2 = ops.w4_linear(xp, t)
            from olmo_amd import _lib
            if _lib.lib().olmo355_gemm_streamk_plan(M, N, K):
                a, b = y2.float(), y[perm.to(dev)].float()
                assert ((a - b).abs() <= 2 ** -7 * torch.maximum(a.abs(), b.abs()) + 2 ** -16 * b.abs().max()).all()
                ops.STREAMK = False
                try:
                    assert torch.equal(ops.w4_linear(xp, t), ops.w4_linear(x.to(dev), t)[perm.to(dev)])
                finally:
                    ops.STREAMK = True
            else:
                assert torch.equal(y2, y[perm.to(dev)])


@pytest.mark.parametrize("N,K", [(4096, 4096), (11008, 4096), (4096, 11008), (13824, 5120), (100352, 4096)])
def test_w4_linear_isolated_sweep_shapes(dev, N, K):
    """Every cell of the isolated sweep (`bench.py --sweep`): M in {1, 8, 64, 512, 4096} on its five (N, K)."""
    say("w4_linear sweep shape", N, K)
    _w4_big_case(dev, N, K, (1, 8, 64, 512, 4096), seed=N + K)


@pytest.mark.parametrize("N,K", [(15360, 5120), (5120, 5120), (27648, 5120), (5120, 13824)])
def test_w4_linear_13b_decode_rows(dev, N, K):
    """The four block Linears of the 13B shape at the 16 rows of its decode batch (and at 4 prefill-sized rows
    counts of the same shapes)."""
    say("w4_linear 13b", N, K)
    _w4_big_case(dev, N, K, (16, 4096), seed=N + K + 1)


@pytest.mark.parametrize("form", [1, 2, 3, 4, 5])
@pytest.mark.parametrize("M,N,K", [(1, 1024, 512), (4, 4096, 4096), (9, 8208, 640), (16, 272, 1408), (40, 2064, 896), (64, 4096, 1024)])
def test_w4_gemv_every_kernel_family(dev, form, M, N, K):
    """Each kernel family the small-M dispatcher chooses between (lean / staged-activation with one or two
    column-tile pairs / the older kernels), forced on shapes it would not have been given, against the oracle."""
    say("w4_gemv form", form, M, N, K)
    ops = _ops()
    from olmo_amd import _lib
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=M + N + K)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16)
    ref = ow4.linear_fp32(x, ow4.dequantize(qw, qz, sc, 128))
    t = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    xd = x.to(dev)
    y = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    st = _lib.lib().olmo355_w4_gemv_form(xd.data_ptr(), t.wt.data_ptr(), t.st.data_ptr(), t.zt.data_ptr(), y.data_ptr(),
                                         M, N, K, form, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert st == 0
    scale = ref.abs().max().item()
    assert (y.float().cpu() - ref).abs().max().item() <= 2 ** -7 * scale


@pytest.mark.parametrize("M", [1, 8, 40, 64, 65, 300, 1024])
@pytest.mark.parametrize("N,K", [(256, 256), (2048, 2048), (1008, 1408)])
def test_b16_linear(dev, M, N, K):
    say("b16_linear", M, N, K)
    ops = _ops()
    gen = torch.Generator().manual_seed(M + N + K)
    w = (torch.randn(N, K, generator=gen) * 0.02).to(torch.bfloat16)
    x = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    ref = x.float() @ w.float().t()
    t = ops.b16_repack(w.to(dev))
    y = ops.b16_linear(x.to(dev), t).float().cpu()
    # exact bf16 products, fp32 accumulation, one bf16 rounding of the result
    assert torch.allclose(y, ref, rtol=2 ** -8, atol=2 ** -8 * ref.abs().max().item())


@pytest.mark.parametrize("M", [1, 8, 65, 300, 1024])
@pytest.mark.parametrize("N,K", [(256, 256), (2048, 2048), (1008, 1408)])
def test_f16_linear(dev, M, N, K):
    say("f16_linear", M, N, K)
    ops = _ops()
    gen = torch.Generator().manual_seed(M + N + K)
    w = (torch.randn(N, K, generator=gen) * 0.02).to(torch.float16)
    x = torch.randn(M, K, generator=gen).to(torch.float16)
    ref = x.float() @ w.float().t()
    t = ops.b16_repack(w.to(dev))
    y = ops.b16_linear(x.to(dev), t)
    assert y.dtype == torch.float16
    # exact fp16 products, fp32 accumulation, one fp16 rounding of the result
    assert torch.allclose(y.float().cpu(), ref, rtol=2 ** -11, atol=2 ** -11 * ref.abs().max().item())
    with pytest.raises(TypeError):
        ops.b16_linear(x.to(dev).bfloat16(), t)


@pytest.mark.parametrize("width", [256, 192, 128, 128128, 128064])
@pytest.mark.parametrize("M,N,K", [(65, 208, 128), (300, 1008, 384), (513, 400, 1408), (256, 768, 256), (1, 16, 640)])
def test_w4_gemm_every_tile_width(dev, width, M, N, K):
    """Ragged M and N against every tile shape, and K whose stage count leaves 0..3 stages after the
    four-stage main loop (int4 stages come in pairs: K = 128, 384, 1408 leave two, 256 none, 640 two)."""
    say("w4_gemm_tile", width, M, N, K)
    ops = _ops()
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=M + N + K)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(7)).to(torch.bfloat16)
    ref = ow4.linear_fp32(x, ow4.dequantize(qw, qz, sc, 128))
    t = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    y = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    xd = x.to(dev)
    from olmo_amd import _lib
    st = _lib.lib().olmo355_w4_gemm_tile(xd.data_ptr(), t.wt.data_ptr(), t.st.data_ptr(), t.zt.data_ptr(), y.data_ptr(),
                                         M, N, K, width, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert st == 0
    scale = ref.abs().max().item()
    assert (y.float().cpu() - ref).abs().max().item() <= 2 ** -7 * scale


STREAMK_STATUS_WORD = 513  # O355_STREAMK_STATUS_WORD of include/olmo355.h


def _streamk_ws(dev):
    from olmo_amd import _lib
    return torch.zeros(_lib.lib().olmo355_gemm_streamk_workspace_bytes(), dtype=torch.uint8, device=dev)


@pytest.mark.parametrize("M,N,K", [(1024, 4096, 1024), (1000, 4080, 1280), (2048, 8192, 512), (700, 6160, 2048),
                                   (2048, 12288, 1024), (1024, 4096, 8448)])
def test_w4_gemm_streamk(dev, M, N, K):
    """The stream-K form against the oracle on shapes where a tile's K is shared by four workgroups (one unit of 256
    per CU), by two with uneven pieces, by none (256 tiles of two units: one whole tile per CU), with ragged M and N,
    and with 1.5 tiles per CU; a second launch on the same workspace, which still holds every flag of the first, with
    the next epoch gives the same bits, and so does a third on a workspace whose flag words were all overwritten with
    a stale epoch (what a launch that was cut short would leave)."""
    say("w4_gemm_streamk", M, N, K)
    from olmo_amd import _lib
    ops = _ops()
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=M + N + K)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(11)).to(torch.bfloat16)
    ref = ow4.linear_fp32(x, ow4.dequantize(qw, qz, sc, 128))
    t = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    xd = x.to(dev)
    ws = _streamk_ws(dev)
    s = torch.cuda.current_stream().cuda_stream
    ys = []
    words = ws.view(torch.int32)
    for epoch in (1, 2, 9):
        if epoch == 9:
            words[:256] = 8  # every hand-over flag left up by an earlier launch
        y = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
        st = _lib.lib().olmo355_w4_gemm_streamk(xd.data_ptr(), t.wt.data_ptr(), t.st.data_ptr(), t.zt.data_ptr(), y.data_ptr(),
                                                M, N, K, ws.data_ptr(), ws.numel(), epoch, s)
        torch.cuda.synchronize()
        assert st == 0
        assert words[STREAMK_STATUS_WORD].item() == 0
        assert set(words[:256].unique().tolist()) <= {0, 8, epoch - 1, epoch}  # flags hold epochs; nothing is cleaned
        ys.append(y)
    assert torch.equal(ys[0], ys[1]) and torch.equal(ys[0], ys[2])
    # a workspace that is too small, or epoch 0, is refused before anything is launched
    args = (xd.data_ptr(), t.wt.data_ptr(), t.st.data_ptr(), t.zt.data_ptr(), ys[0].data_ptr(), M, N, K, ws.data_ptr())
    assert _lib.lib().olmo355_w4_gemm_streamk(*args, ws.numel() - 1, 10, s) == 1
    assert _lib.lib().olmo355_w4_gemm_streamk(*args, ws.numel(), 0, s) == 1
    scale = ref.abs().max().item()
    assert (ys[0].float().cpu() - ref).abs().max().item() <= 2 ** -7 * scale
    # against the tiled launch: the same fp32 products added in another order
    y0 = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    assert _lib.lib().olmo355_w4_gemm(xd.data_ptr(), t.wt.data_ptr(), t.st.data_ptr(), t.zt.data_ptr(), y0.data_ptr(), M, N, K, s) == 0
    torch.cuda.synchronize()
    a, b = ys[0].float(), y0.float()  # one rounding step of the element, or what fp32 sums of this size differ by near zero
    assert ((a - b).abs() <= 2 ** -7 * torch.maximum(a.abs(), b.abs()) + 2 ** -16 * scale).all()


def test_w4_gemm_swiglu_streamk_and_dense_streamk(dev):
    """The SwiGLU-epilogue and dense forms of the stream-K launch against their tiled counterparts."""
    say("w4_gemm_swiglu_streamk / b16_gemm_streamk")
    from olmo_amd import _lib
    ops = _ops()
    L = _lib.lib()
    M, N, K = 1100, 8192, 1024
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=77)
    t = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(12)).to(torch.bfloat16).to(dev)
    ws = _streamk_ws(dev)
    s = torch.cuda.current_stream().cuda_stream
    y0 = torch.empty(M, N // 2, dtype=torch.bfloat16, device=dev)
    y1 = torch.full_like(y0, float("nan"))
    assert L.olmo355_w4_gemm_swiglu(x.data_ptr(), t.wt.data_ptr(), t.st.data_ptr(), t.zt.data_ptr(), y0.data_ptr(), M, N, K, s) == 0
    assert L.olmo355_w4_gemm_swiglu_streamk(x.data_ptr(), t.wt.data_ptr(), t.st.data_ptr(), t.zt.data_ptr(), y1.data_ptr(), M, N, K,
                                            ws.data_ptr(), ws.numel(), 1, s) == 0
    torch.cuda.synchronize()
    a, b = y1.float(), y0.float()
    # silu(gate) * up of two bf16-rounded factors: one rounding step of either factor moves the product by 2^-7
    assert ((a - b).abs() <= 2 ** -6 * torch.maximum(a.abs(), b.abs()) + 2 ** -14 * b.abs().max()).all()
    assert ws.view(torch.int32)[STREAMK_STATUS_WORD].item() == 0
    w = (torch.randn(N, K, generator=torch.Generator().manual_seed(13)) * 0.02).to(torch.bfloat16).to(dev)
    tw = ops.b16_repack(w)
    z0 = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    z1 = torch.full_like(z0, float("nan"))
    assert L.olmo355_b16_gemm(x.data_ptr(), tw.wt.data_ptr(), z0.data_ptr(), M, N, K, s) == 0
    assert L.olmo355_b16_gemm_streamk(x.data_ptr(), tw.wt.data_ptr(), z1.data_ptr(), M, N, K, ws.data_ptr(), ws.numel(), 2,
                                      s) == 0
    torch.cuda.synchronize()
    a, b = z1.float(), z0.float()
    assert ((a - b).abs() <= 2 ** -7 * torch.maximum(a.abs(), b.abs()) + 2 ** -16 * b.abs().max()).all()
    ref = x.float() @ w.float().t()
    assert torch.allclose(z1.float(), ref, rtol=2 ** -8, atol=2 ** -8 * ref.abs().max().item())


def test_w4_gemm_streamk_gives_up_instead_of_hanging(dev):
    """With the partials' owners told not to raise their flags (a host-side switch of the variant entry) and a
    patience of four polls, every finishing workgroup gives its tile up as NaN, the tiles that were never shared are
    right, the launch ends with its epoch in the status word, and the next launch on the same workspace, not cleaned,
    is right."""
    say("w4_gemm_streamk give-up")
    from olmo_amd import _lib
    ops = _ops()
    L = _lib.lib()
    M, N, K = 2048, 12288, 1024  # 384 tiles on 256 CUs: every second tile is shared by two workgroups
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=5)
    t = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(14)).to(torch.bfloat16).to(dev)
    ws = _streamk_ws(dev)
    s = torch.cuda.current_stream().cuda_stream
    y = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    st = L.olmo355_w4_gemm_streamk_patience(x.data_ptr(), t.wt.data_ptr(), t.st.data_ptr(), t.zt.data_ptr(), y.data_ptr(),
                                            M, N, K, ws.data_ptr(), ws.numel(), 5, 4, 0, s)
    torch.cuda.synchronize()
    assert st == 0
    assert ws.view(torch.int32)[STREAMK_STATUS_WORD].item() == 5
    y0 = torch.empty_like(y)
    assert L.olmo355_w4_gemm(x.data_ptr(), t.wt.data_ptr(), t.st.data_ptr(), t.zt.data_ptr(), y0.data_ptr(), M, N, K, s) == 0
    torch.cuda.synchronize()
    tiles = y.float().view(M // 256, 256, N // 256, 256).permute(0, 2, 1, 3).reshape(-1, 256 * 256)
    ref_tiles = y0.float().view(M // 256, 256, N // 256, 256).permute(0, 2, 1, 3).reshape(-1, 256 * 256)
    nan_tiles = torch.isnan(tiles).all(dim=1)
    clean = ~torch.isnan(tiles).any(dim=1)
    assert (nan_tiles | clean).all()                     # a tile is given up whole or not at all
    assert nan_tiles.sum().item() == 128 and clean.sum().item() == 256
    assert torch.equal(tiles[clean], ref_tiles[clean])   # whole tiles: the same additions in the same order as the tiled launch
    # the workspace as the failed launch left it serves the next one
    y2 = torch.full_like(y, float("nan"))
    assert L.olmo355_w4_gemm_streamk(x.data_ptr(), t.wt.data_ptr(), t.st.data_ptr(), t.zt.data_ptr(), y2.data_ptr(), M, N, K,
                                     ws.data_ptr(), ws.numel(), 6, s) == 0
    torch.cuda.synchronize()
    a, b = y2.float(), y0.float()
    assert ((a - b).abs() <= 2 ** -7 * torch.maximum(a.abs(), b.abs()) + 2 ** -16 * b.abs().max()).all()
    assert ws.view(torch.int32)[STREAMK_STATUS_WORD].item() == 5  # kept until its reader clears it


def test_gemm_rejects_misaligned_output(dev):
    """The matrix-core epilogue stores 16 bytes per lane: an output that does not start on a 16-byte boundary is
    refused (status 1, nothing launched); the same call on the aligned buffer runs."""
    from olmo_amd import _lib
    ops = _ops()
    M, N, K = 65, 64, 128
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=3)
    t = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    x = torch.randn(M, K, device=dev).to(torch.bfloat16)
    buf = torch.zeros(M * N + 8, dtype=torch.bfloat16, device=dev)
    s = torch.cuda.current_stream().cuda_stream
    st = _lib.lib().olmo355_w4_gemm(x.data_ptr(), t.wt.data_ptr(), t.st.data_ptr(), t.zt.data_ptr(), buf.data_ptr() + 2,
                                    M, N, K, s)
    torch.cuda.synchronize()
    assert st == 1 and not buf.any()
    st = _lib.lib().olmo355_w4_gemm(x.data_ptr(), t.wt.data_ptr(), t.st.data_ptr(), t.zt.data_ptr(), buf.data_ptr(), M, N, K, s)
    torch.cuda.synchronize()
    assert st == 0 and buf.any()


@pytest.mark.parametrize("width", [256, 192, 128, 128128, 128064])
@pytest.mark.parametrize("M,N,K", [(65, 208, 64), (300, 1008, 192), (513, 400, 320), (256, 768, 448), (40, 48, 1024)])
def test_b16_gemm_every_tile_width(dev, width, M, N, K):
    """Dense weights: stage counts 1, 3, 5, 7, 16 cover every tail length of the four-stage loop."""
    say("b16_gemm_tile", width, M, N, K)
    ops = _ops()
    gen = torch.Generator().manual_seed(M + N + K)
    w = (torch.randn(N, K, generator=gen) * 0.02).to(torch.bfloat16)
    x = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    ref = x.float() @ w.float().t()
    t = ops.b16_repack(w.to(dev))
    y = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    xd = x.to(dev)
    from olmo_amd import _lib
    st = _lib.lib().olmo355_b16_gemm_tile(xd.data_ptr(), t.wt.data_ptr(), y.data_ptr(), M, N, K, width,
                                          torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert st == 0
    assert torch.allclose(y.float().cpu(), ref, rtol=2 ** -8, atol=2 ** -8 * ref.abs().max().item())


@pytest.mark.parametrize("splits", [2, 3, 5])
@pytest.mark.parametrize("M,N,K", [(65, 64, 1536), (128, 4096, 2816), (300, 1024, 1280), (512, 256, 4096), (33, 384, 1280),
                                   (64, 4096, 2816)])
def test_gemm_splitk(dev, splits, M, N, K):
    """Several workgroups per tile along K (int4 and dense): uneven runs (K / 256 = 6, 11, 5, 16 units over 2, 3, 5
    splits), ragged M, runs as short as one unit; against the oracle product and against the plain entry (same
    products, other order of the fp32 additions: equal up to one rounding of the bf16 result)."""
    say("gemm_splitk", splits, M, N, K)
    ops = _ops()
    from olmo_amd import _lib
    L = _lib.lib()
    s_ = torch.cuda.current_stream().cuda_stream
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=M + N + K)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(7)).to(torch.bfloat16)
    ref = ow4.linear_fp32(x, ow4.dequantize(qw, qz, sc, 128))
    t = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    xd = x.to(dev)
    y = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    y0 = torch.empty_like(y)
    part = torch.empty(splits, M, N, dtype=torch.float32, device=dev)
    assert L.olmo355_w4_gemm_splitk(xd.data_ptr(), t.wt.data_ptr(), t.st.data_ptr(), t.zt.data_ptr(), y.data_ptr(), M, N, K,
                                    splits, part.data_ptr(), s_) == 0
    assert L.olmo355_w4_gemm(xd.data_ptr(), t.wt.data_ptr(), t.st.data_ptr(), t.zt.data_ptr(), y0.data_ptr(), M, N, K, s_) == 0
    torch.cuda.synchronize()
    scale = ref.abs().max().item()
    assert (y.float().cpu() - ref).abs().max().item() <= 2 ** -7 * scale
    assert (y.float() - y0.float()).abs().max().item() <= 2 ** -7 * scale
    assert (y == y0).float().mean().item() > 0.9
    # the partial sums add up to the product in fp32
    assert (part.sum(0).cpu() - ref).abs().max().item() <= 2e-5 * scale * (K / 128) ** 0.5 + 2 ** -9 * scale
    # dense
    g = torch.Generator().manual_seed(M + N + K)
    w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
    refd = x.float() @ w.float().t()
    td = ops.b16_repack(w.to(dev))
    assert L.olmo355_b16_gemm_splitk(xd.data_ptr(), td.wt.data_ptr(), y.data_ptr(), M, N, K, splits, part.data_ptr(), s_) == 0
    torch.cuda.synchronize()
    assert torch.allclose(y.float().cpu(), refd, rtol=2 ** -8, atol=2 ** -8 * refd.abs().max().item())
    assert (part.sum(0).cpu() - refd).abs().max().item() <= 1e-4 * refd.abs().max().item()


def test_gemm_splitk_plan_and_routing(dev):
    """The plan splits only when tiles are scarce, and ops.w4_linear follows it."""
    say("gemm_splitk plan")
    ops = _ops()
    from olmo_amd import _lib
    plan = _lib.lib().olmo355_gemm_splitk_plan
    assert plan(64, 4096, 4096) == 1 and plan(2048, 4096, 4096) == 1 and plan(128, 4096, 4000) == 1
    assert plan(64, 4096, 11008) == 8 and plan(33, 4096, 11008) == 8 and plan(32, 4096, 11008) == 1 and plan(64, 12288, 11008) == 1
    assert plan(128, 4096, 4096) == 4 and plan(512, 4096, 4096) == 1 and plan(128, 4096, 11008) == 8
    assert plan(512, 4096, 11008) == 2 and plan(256, 4096, 11008) == 4
    assert plan(128, 22016, 4096) == 1 and plan(128, 12288, 4096) == 2 and plan(300, 4096, 4096) == 2
    qw, qz, sc = ow4.random_quantized(2048, 1024, 128, seed=3)
    t = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    x = torch.randn(130, 2048, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).to(dev)
    assert plan(130, 1024, 2048) == 2
    a = ops.w4_linear(x, t)
    ops.SPLITK = False
    try:
        b = ops.w4_linear(x, t)
    finally:
        ops.SPLITK = True
    ref = ow4.linear_fp32(x.cpu(), ow4.dequantize(qw, qz, sc, 128))
    scale = ref.abs().max().item()
    assert (a.float().cpu() - ref).abs().max().item() <= 2 ** -7 * scale
    assert (b.float().cpu() - ref).abs().max().item() <= 2 ** -7 * scale


@pytest.mark.parametrize("M,N,K", [(1, 50304, 256), (2048, 768, 256), (77, 130, 1024)])
def test_f32_linear(dev, M, N, K):
    ops = _ops()
    gen = torch.Generator().manual_seed(M + N)
    w = torch.randn(N, K, generator=gen) * 0.02
    x = torch.randn(M, K, generator=gen)
    ref = (x.double() @ w.double().t()).float()
    y = ops.f32_linear(x.to(dev), w.to(dev)).cpu()
    assert torch.allclose(y, ref, rtol=1e-5, atol=1e-5)


# ------------------------------------------------------------------------------------------------
# row kernels
# ------------------------------------------------------------------------------------------------
_MANT = {torch.bfloat16: 7, torch.float16: 10}  # stored mantissa bits of the 16-bit activation dtypes
_ACT_DTYPES = [torch.float32, torch.bfloat16, torch.float16]


@pytest.mark.parametrize("dtype", _ACT_DTYPES)
@pytest.mark.parametrize("rows,d", [(1, 4096), (37, 2048), (5, 5120), (3, 256)])
def test_rmsnorm(dev, dtype, rows, d):
    ops = _ops()
    gen = torch.Generator().manual_seed(rows + d)
    x = (torch.randn(rows, d, generator=gen) * 3).to(dtype)
    w = (1 + 0.1 * torch.randn(d, generator=gen)).to(dtype)
    r = torch.randn(rows, d, generator=gen).to(dtype)
    ref = om.rms_norm(x, w, 1e-6)
    out = ops.rmsnorm(x.to(dev), w.to(dev), 1e-6).cpu()
    out_r = ops.rmsnorm(x.to(dev), w.to(dev), 1e-6, residual=r.to(dev)).cpu()
    if dtype == torch.float32:
        assert torch.allclose(out, ref, rtol=1e-5, atol=1e-6)
        assert torch.allclose(out_r, r + ref, rtol=1e-5, atol=1e-5)
    else:
        # same rounding points; the fp32 sum of squares may differ in the last bit, which can
        # flip a rounding: allow 1 ulp of the dtype on at most 0.5% of the elements
        diff = (out.float() - ref.float()).abs()
        ulp = 2.0 ** (torch.floor(torch.log2(ref.float().abs().clamp_min(1e-30))) - _MANT[dtype])
        assert (diff <= ulp).all()
        assert (diff > 0).float().mean().item() < 5e-3
        assert (out_r.float() - (r + ref).float()).abs().max().item() <= 2 * ulp.max().item()


@pytest.mark.parametrize("dtype", _ACT_DTYPES)
@pytest.mark.parametrize("rows,d", [(1, 4096), (8, 5120), (3, 256), (2, 8192)])
def test_rmsnorm_pair_equals_the_two_norms(dev, dtype, rows, d):
    """The one-launch form of a decode step's last two norms, bit for bit against the two launches it replaces (which
    test_rmsnorm holds against the oracle); a width it does not take is declined."""
    ops = _ops()
    gen = torch.Generator().manual_seed(rows + d)
    if dtype == torch.float32 and d > 4096:
        d = 4096
    x = (torch.randn(rows, d, generator=gen) * 3).to(dtype).to(dev)
    r = torch.randn(rows, d, generator=gen).to(dtype).to(dev)
    w1 = (1 + 0.1 * torch.randn(d, generator=gen)).to(dtype).to(dev)
    w2 = (1 + 0.1 * torch.randn(d, generator=gen)).to(dtype).to(dev)
    two = ops.rmsnorm(ops.rmsnorm(x, w1, 1e-6, residual=r), w2, 1e-6)
    one = ops.rmsnorm_pair(x, w1, r, w2, 1e-6)
    assert one is not None and torch.equal(one, two)
    odd = torch.randn(2, 1002, generator=gen).to(dtype).to(dev)
    wo = torch.ones(1002, dtype=dtype, device=dev)
    assert ops.rmsnorm_pair(odd, wo, odd, wo, 1e-6) is None


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("rows,n", [(1, 100352), (8, 100352), (3, 1003)])
def test_greedy_next_equals_argmax_embedding_and_rope_advance(dev, dtype, rows, n):
    """The one-launch end of a greedy decode step against the three launches it replaces: tokens (ties: first index),
    embedding rows of the chosen tokens, position and rotary rows; a table with fewer rows than the logits are wide
    reads its last row for ids past it."""
    ops = _ops()
    gen = torch.Generator().manual_seed(rows + n)
    lg = torch.randn(rows, n, generator=gen).to(dtype)
    lg[0, 77] = lg[0, 900] = 9.0
    if rows > 1:
        lg[1, n - 1] = 11.0  # past a table of n - 5 rows
    lg = lg.to(dev)
    d, hd, n_pos = 520, 64, 40
    tab = torch.randn(n - 5, d, generator=gen).to(dtype).to(dev)
    sin, cos = ops.rope_tables(hd, 10000.0, n_pos, dev)
    for start in (0, 17, n_pos - 1):  # the last: the position runs past the table, its last row stays
        pos_a = torch.full((1,), start, dtype=torch.int32, device=dev)
        pos_b = pos_a.clone()
        now_a = torch.zeros(2 * hd, dtype=torch.float32, device=dev)
        now_b = torch.zeros_like(now_a)
        ids_a = ops.argmax(lg)
        x_a = ops.embedding(ids_a, tab)
        ops.rope_advance(pos_a, 1, sin, cos, now_a)
        ids_b = torch.full((rows,), -1, dtype=torch.int64, device=dev)
        x_b = torch.full((rows, d), float("nan"), dtype=dtype, device=dev)
        ops.greedy_next(lg, ids_b, tab, x_b, pos_b, sin, cos, now_b)
        assert torch.equal(ids_a, ids_b) and int(ids_b[0]) == 77
        assert torch.equal(x_a.view(rows, d), x_b)
        assert torch.equal(pos_a, pos_b) and int(pos_b) == start + 1 and torch.equal(now_a, now_b)


@pytest.mark.parametrize("rows,d", [(2048, 256), (3, 1000)])
def test_layernorm_np(dev, rows, d):
    ops = _ops()
    x = torch.randn(rows, d, generator=torch.Generator().manual_seed(d)) * 2 + 0.5
    ref = om.layer_norm_np(x, 1e-5)
    out = ops.layernorm_np(x.to(dev), 1e-5).cpu()
    assert torch.allclose(out, ref, rtol=1e-5, atol=2e-6)


@pytest.mark.parametrize("dtype", _ACT_DTYPES)
def test_swiglu(dev, dtype):
    ops = _ops()
    x = (torch.randn(33, 2 * 1376, generator=torch.Generator().manual_seed(4)) * 2).to(dtype)
    ref = om.swiglu(x)
    out = ops.swiglu(x.to(dev)).cpu()
    if dtype == torch.float32:
        assert torch.allclose(out, ref, rtol=1e-5, atol=1e-6)
    else:
        diff = (out.float() - ref.float()).abs()
        ulp = 2.0 ** (torch.floor(torch.log2(ref.float().abs().clamp_min(1e-30))) - _MANT[dtype])
        assert (diff <= ulp).all() and (diff > 0).float().mean().item() < 5e-3


def test_embedding_add_argmax(dev):
    ops = _ops()
    gen = torch.Generator().manual_seed(0)
    tab = torch.randn(1000, 256, generator=gen).to(torch.bfloat16)
    ids = torch.randint(0, 1000, (3, 7), generator=gen)
    assert torch.equal(ops.embedding(ids.to(dev), tab.to(dev)).cpu(), tab[ids])
    a, b = torch.randn(5, 100, generator=gen).bfloat16(), torch.randn(5, 100, generator=gen).bfloat16()
    assert torch.equal(ops.add(a.to(dev), b.to(dev)).cpu(), a + b)
    lg = torch.randn(4, 100352, generator=gen).bfloat16()
    lg[1, 77] = lg[1, 5000] = 9.0  # tie: first index wins
    assert torch.equal(ops.argmax(lg.to(dev)).cpu(), torch.argmax(lg.float(), dim=-1))
    assert int(ops.argmax(lg.to(dev))[1]) == 77
    # the same in fp16
    th, ah, bh, lh = tab.half(), a.half(), b.half(), lg.half()
    assert torch.equal(ops.embedding(ids.to(dev), th.to(dev)).cpu(), th[ids])
    assert torch.equal(ops.add(ah.to(dev), bh.to(dev)).cpu(), (ah.float() + bh.float()).half())
    assert torch.equal(ops.argmax(lh.to(dev)).cpu(), torch.argmax(lh.float(), dim=-1))
    xc = (torch.randn(7, 300, generator=gen) * 3).half()
    assert torch.equal(ops.clamp_(xc.to(dev), 1.5).cpu(), xc.clamp(-1.5, 1.5))


# ------------------------------------------------------------------------------------------------
# attention path
# ------------------------------------------------------------------------------------------------
def _rope_ref(qkv, qw, kw, B, T, H, Hkv, hd, past, theta, eps, n_pos):
    dq, dk = H * hd, Hkv * hd
    q, k, v = qkv.view(B, T, -1).split((dq, dk, dk), dim=-1)
    if qw is not None:
        q, k = om.rms_norm(q, qw, eps), om.rms_norm(k, kw, eps)
    q = q.reshape(B, T, H, hd).transpose(1, 2)
    k = k.reshape(B, T, Hkv, hd).transpose(1, 2)
    v = v.reshape(B, T, Hkv, hd).transpose(1, 2)
    sin, cos = om.rope_tables(hd, theta, n_pos)
    q = om.apply_rope(q, sin[past:past + T], cos[past:past + T])
    k = om.apply_rope(k, sin[past:past + T], cos[past:past + T])
    return q, k, v


@pytest.mark.parametrize("dtype,qknorm,H,Hkv,hd", [(torch.bfloat16, True, 16, 16, 128), (torch.bfloat16, True, 8, 2, 64),
                                                    (torch.float32, False, 8, 8, 32), (torch.float16, True, 8, 2, 64),
                                                    (torch.float16, False, 4, 4, 128)])
def test_qknorm_rope_kvwrite(dev, dtype, qknorm, H, Hkv, hd):
    ops = _ops()
    B, T, past, Lmax, theta, eps = 2, 5, 3, 16, 500000.0, 1e-6
    gen = torch.Generator().manual_seed(hd)
    qkv = torch.randn(B * T, (H + 2 * Hkv) * hd, generator=gen).to(dtype)
    qw = (1 + 0.1 * torch.randn(H * hd, generator=gen)).to(dtype) if qknorm else None
    kw = (1 + 0.1 * torch.randn(Hkv * hd, generator=gen)).to(dtype) if qknorm else None
    qr, kr, vr = _rope_ref(qkv, qw, kw, B, T, H, Hkv, hd, past, theta, eps, Lmax)
    sin, cos = ops.rope_tables(hd, theta, Lmax, dev)
    kc = torch.zeros(B, Hkv, Lmax, hd, dtype=dtype, device=dev)
    vc = torch.zeros_like(kc)
    q = ops.qknorm_rope_kvwrite(qkv.to(dev), None if qw is None else qw.to(dev), None if kw is None else kw.to(dev),
                                sin, cos, kc, vc, B, T, H, Hkv, hd, past, eps)
    q = q.view(B, T, H, hd).transpose(1, 2).cpu()
    tol = {torch.float32: dict(rtol=1e-5, atol=1e-5), torch.bfloat16: dict(rtol=2 ** -7, atol=2 ** -7),
           torch.float16: dict(rtol=2 ** -10, atol=2 ** -10)}[dtype]
    assert torch.allclose(q.float(), qr.float(), **tol)
    assert torch.allclose(kc[:, :, past:past + T].cpu().float(), kr.float(), **tol)
    assert torch.equal(vc[:, :, past:past + T].cpu(), vr)
    assert (kc[:, :, :past] == 0).all() and (kc[:, :, past + T:] == 0).all()
    if dtype != torch.float32:  # same rounding points: almost every element identical
        assert (q.float() != qr.float()).float().mean().item() < 1e-2


@pytest.mark.parametrize("dtype,B,T,past,H,Hkv,hd", [
    (torch.bfloat16, 1, 300, 0, 4, 4, 128),
    (torch.bfloat16, 2, 130, 70, 4, 2, 128),
    (torch.bfloat16, 1, 257, 0, 2, 2, 64),
    # one query; a tile short of / exactly / just over one key tile and one query block; a long past; many tiles
    (torch.bfloat16, 1, 1, 0, 2, 2, 128),
    (torch.bfloat16, 1, 63, 0, 2, 2, 128),
    (torch.bfloat16, 2, 64, 0, 2, 1, 64),
    (torch.bfloat16, 2, 65, 5, 4, 4, 64),
    (torch.bfloat16, 1, 128, 0, 2, 2, 128),
    (torch.bfloat16, 1, 129, 127, 2, 1, 128),
    (torch.bfloat16, 1, 7, 1000, 2, 2, 128),
    (torch.bfloat16, 1, 1000, 24, 2, 2, 128),
    (torch.bfloat16, 1, 1000, 24, 2, 2, 64),
    (torch.float32, 2, 100, 0, 8, 8, 32),
    (torch.float32, 1, 70, 30, 2, 2, 32),
    # prompts from scratch of more than 1024 tokens: the long query blocks are shared between workgroups along the keys
    # (two, two with a ragged last block, three and four runs of keys per block)
    (torch.bfloat16, 1, 2048, 0, 4, 4, 128),
    (torch.bfloat16, 1, 1153, 0, 2, 1, 128),
    (torch.bfloat16, 2, 3000, 0, 2, 2, 64),
    (torch.bfloat16, 1, 4096, 0, 2, 2, 128),
    # fp16 activations: every head size on the one-thread-per-row kernel
    (torch.float16, 1, 300, 0, 4, 4, 128),
    (torch.float16, 2, 130, 70, 4, 2, 64),
    (torch.float16, 1, 70, 30, 2, 2, 32),
    (torch.float16, 1, 1500, 0, 2, 2, 128),
])
def test_attn_prefill(dev, dtype, B, T, past, H, Hkv, hd):
    say("attn_prefill", dtype, B, T, past, H, Hkv, hd)
    ops = _ops()
    L = past + T
    Lmax = L + 9
    gen = torch.Generator().manual_seed(T + hd)
    q = torch.randn(B, H, T, hd, generator=gen).to(dtype)
    k = torch.randn(B, Hkv, L, hd, generator=gen).to(dtype)
    v = torch.randn(B, Hkv, L, hd, generator=gen).to(dtype)
    ref = om.attention(q, k, v, None, dtype).transpose(1, 2).reshape(B, T, H * hd)
    kc = torch.zeros(B, Hkv, Lmax, hd, dtype=dtype)
    vc = torch.zeros_like(kc)
    kc[:, :, :L], vc[:, :, :L] = k, v
    poison_lds(dev)
    out = ops.attn_prefill(q.transpose(1, 2).reshape(B, T, H * hd).contiguous().to(dev), kc.to(dev), vc.to(dev), B, T, H,
                           Hkv, hd, past).cpu()
    if dtype == torch.float32:
        assert torch.allclose(out, ref, rtol=1e-4, atol=1e-5)
    elif dtype == torch.float16:  # fp32 arithmetic on the widened operands, one rounding of the output
        assert torch.allclose(out.float(), ref.float(), rtol=2 ** -10, atol=2 ** -12)
    else:
        # P is rounded to bf16 before the second product (2^-9 relative), output rounded to bf16
        assert torch.allclose(out.float(), ref.float(), rtol=0, atol=2.5e-2)
        assert (out.float() - ref.float()).abs().mean().item() < 2e-3
    # padding: mask the first 5 keys of batch row 0 (left padding)
    bias = torch.zeros(B, Lmax)
    bias[0, :5] = torch.finfo(torch.float32).min
    fb = torch.triu(torch.ones(L, L), diagonal=1).masked_fill_(torch.triu(torch.ones(L, L), diagonal=1) == 1,
                                                               torch.finfo(torch.float32).min).view(1, 1, L, L)
    fb = (fb + bias[:, None, None, :L])
    fb = fb.masked_fill(fb == float("-inf"), torch.finfo(torch.float32).min)[:, :, L - T:L]
    fb = fb.to(dtype)
    fb = fb.masked_fill(fb == float("-inf"), torch.finfo(dtype).min)
    ref2 = om.attention(q, k, v, fb, dtype).transpose(1, 2).reshape(B, T, H * hd)
    poison_lds(dev)
    out2 = ops.attn_prefill(q.transpose(1, 2).reshape(B, T, H * hd).contiguous().to(dev), kc.to(dev), vc.to(dev), B, T,
                            H, Hkv, hd, past, key_bias=bias.to(dev)).cpu()
    valid = slice(5, None) if past == 0 else slice(None)  # rows that see at least one real key
    tol = {torch.float32: dict(rtol=1e-4, atol=1e-5), torch.bfloat16: dict(rtol=0, atol=2.5e-2),
           torch.float16: dict(rtol=2 ** -10, atol=2 ** -12)}[dtype]
    assert torch.allclose(out2[:, valid].float(), ref2[:, valid].float(), **tol)
    assert torch.isfinite(out2.float()).all()
    from olmo_amd import _lib
    if _lib.lib().olmo355_attn_prefill_workspace_bytes(B, T, H, hd, past, ops._DT[dtype]):
        # the key-split form ran above (twice on one workspace: its counters must have come back to zero); the plain
        # launch forms the same products and differs only in how a row's partial sums are combined
        qd = q.transpose(1, 2).reshape(B, T, H * hd).contiguous().to(dev)
        again = ops.attn_prefill(qd, kc.to(dev), vc.to(dev), B, T, H, Hkv, hd, past).cpu()
        assert torch.equal(again, out)
        ops.PREFILL_SPLIT = False
        try:
            plain = ops.attn_prefill(qd, kc.to(dev), vc.to(dev), B, T, H, Hkv, hd, past).cpu()
        finally:
            ops.PREFILL_SPLIT = True
        a, b = out.float(), plain.float()
        assert ((a - b).abs() <= 2 ** -7 * torch.maximum(a.abs(), b.abs()) + 2 ** -9).all()
        assert not torch.equal(a, b) or T <= 1024  # the two forms really are different launches


@pytest.mark.parametrize("dtype,B,L,H,Hkv,hd", [
    (torch.bfloat16, 1, 2048, 32, 32, 128),   # 48 keys per wave
    (torch.bfloat16, 3, 700, 4, 2, 128),      # 32 keys per wave
    (torch.bfloat16, 8, 1300, 32, 32, 128),   # 64 keys per wave (many heads x sequences)
    (torch.float32, 16, 1100, 8, 8, 32),      # the same in fp32
    (torch.bfloat16, 2, 1, 2, 2, 64),
    (torch.bfloat16, 2, 257, 2, 2, 64),
    (torch.float32, 2, 513, 8, 8, 32),
    (torch.float16, 3, 700, 4, 2, 128),
    (torch.float16, 2, 257, 2, 2, 64),
    (torch.float16, 16, 1100, 8, 8, 32),
])
def test_attn_decode(dev, dtype, B, L, H, Hkv, hd):
    say("attn_decode", dtype, B, L, H, Hkv, hd)
    ops = _ops()
    Lmax = L + 100
    gen = torch.Generator().manual_seed(L + hd)
    q = torch.randn(B, H, 1, hd, generator=gen).to(dtype)
    k = torch.randn(B, Hkv, L, hd, generator=gen).to(dtype)
    v = torch.randn(B, Hkv, L, hd, generator=gen).to(dtype)
    ref = om.attention(q, k, v, None, dtype).transpose(1, 2).reshape(B, 1, H * hd)
    kc = torch.zeros(B, Hkv, Lmax, hd, dtype=dtype)
    vc = torch.zeros_like(kc)
    kc[:, :, :L], vc[:, :, :L] = k, v
    kc, vc = kc.to(dev), vc.to(dev)
    qd = q.reshape(B, 1, H * hd).contiguous().to(dev)
    ws = ops.attn_decode_workspace(B, H, hd, Lmax, dev)
    tol = {torch.float32: dict(rtol=1e-4, atol=1e-5), torch.bfloat16: dict(rtol=2 ** -7, atol=2 ** -8),
           torch.float16: dict(rtol=2 ** -10, atol=2 ** -12)}[dtype]
    out = ops.attn_decode(qd, kc, vc, ws, B, H, Hkv, hd, L - 1, L).cpu()
    assert torch.allclose(out.float(), ref.float(), **tol)
    # position read from device memory, launch grid sized for the whole cache
    pl = torch.tensor([L - 1], dtype=torch.int32, device=dev)
    out_d = ops.attn_decode(qd, kc, vc, ws, B, H, Hkv, hd, 0, Lmax, past_len_dev=pl).cpu()
    assert torch.equal(out_d, out)
    # padding mask on batch row 0
    if L > 8:
        bias = torch.zeros(B, Lmax)
        bias[0, :5] = torch.finfo(torch.float32).min
        fb = bias[:, None, None, :L].to(dtype)
        fb = fb.masked_fill(fb == float("-inf"), torch.finfo(dtype).min)
        ref2 = om.attention(q, k, v, fb, dtype).transpose(1, 2).reshape(B, 1, H * hd)
        out2 = ops.attn_decode(qd, kc, vc, ws, B, H, Hkv, hd, L - 1, L, key_bias=bias.to(dev)).cpu()
        assert torch.allclose(out2.float(), ref2.float(), **tol)


# ------------------------------------------------------------------------------------------------
# decode-step fusions: x' = resid + rmsnorm(a) in the prologue, SwiGLU in the epilogue
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("quant", [True, False])
@pytest.mark.parametrize("M", [1, 3, 8, 16])
@pytest.mark.parametrize("N,K,pro,epi", [(768, 256, True, False), (1024, 256, True, True), (12288, 4096, True, False),
                                         (22016, 4096, True, True), (22016, 4096, False, True), (16384, 2048, True, True)])
def test_linear_fused(dev, quant, M, N, K, pro, epi):
    say("linear_fused", quant, M, N, K, pro, epi)
    ops = _ops()
    gen = torch.Generator().manual_seed(M + N + K)
    a = (torch.randn(M, K, generator=gen) * 2).to(torch.bfloat16)
    resid = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    nw = (1 + 0.1 * torch.randn(K, generator=gen)).to(torch.bfloat16)
    if quant:
        qw, qz, sc = ow4.random_quantized(K, N, 128, seed=N + K)
        Wf = ow4.dequantize(qw, qz, sc, 128).float()  # [K,N]
        w = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    else:
        wd = (torch.randn(N, K, generator=gen) * 0.02).to(torch.bfloat16)
        Wf = wd.float().t()
        w = ops.b16_repack(wd.to(dev))
    x_ref = (resid + om.rms_norm(a, nw, 1e-6)) if pro else a
    y_ref = (x_ref.float() @ Wf).to(torch.bfloat16)
    if epi:
        y_ref = om.swiglu(y_ref)
    y, x_new = ops.linear_fused(a.to(dev), w, resid=resid.to(dev) if pro else None, norm_w=nw.to(dev) if pro else None,
                                eps=1e-6, swiglu_out=epi)
    y, x_new = y.cpu(), x_new.cpu()
    assert y.shape == y_ref.shape
    # x': same rounding points as the separate kernel (1 bf16 ulp where the fp32 sum of squares differs)
    dx = (x_new.float() - x_ref.float()).abs()
    assert (dx <= 2.0 ** (torch.floor(torch.log2(x_ref.float().abs().clamp_min(1e-30))) - 7)).all()
    scale = y_ref.float().abs().max().item()
    assert (y.float() - y_ref.float()).abs().max().item() <= 2 ** -6 * scale
    # and equal to the unfused sequence of kernels up to the last bit of each rounding
    x2 = ops.rmsnorm(a.to(dev), nw.to(dev), 1e-6, residual=resid.to(dev)) if pro else a.to(dev)
    y2 = ops.w4_linear(x2, w) if quant else ops.b16_linear(x2, w)
    y2 = (ops.swiglu(y2) if epi else y2).cpu()
    assert (y.float() - y2.float()).abs().max().item() <= 2 ** -6 * scale


@pytest.mark.parametrize("qknorm,B,past,H,Hkv,hd", [(True, 1, 2048, 32, 32, 128), (True, 3, 700, 4, 2, 128),
                                                     (False, 2, 0, 2, 2, 64), (True, 2, 127, 8, 8, 64),
                                                     (True, 2, 128, 4, 4, 128),
                                                     # more than 1536 workgroups: partials + the separate combine
                                                     # kernel (batch 8 at context 2048 of the 7B shape; 13B heads at 4090)
                                                     (True, 8, 2048, 32, 32, 128), (True, 3, 4090, 40, 40, 128)])
def test_attn_decode_fused(dev, qknorm, B, past, H, Hkv, hd):
    """QK-norm + rotary + cache append + attention in one pass == the two separate kernels == the oracle."""
    say("attn_decode_fused", qknorm, B, past, H, Hkv, hd)
    ops = _ops()
    dtype, theta, eps = torch.bfloat16, 500000.0, 1e-6
    Lmax = past + 200
    gen = torch.Generator().manual_seed(past + hd + H)
    qkv = torch.randn(B, (H + 2 * Hkv) * hd, generator=gen).to(dtype)
    qw = (1 + 0.1 * torch.randn(H * hd, generator=gen)).to(dtype) if qknorm else None
    kw = (1 + 0.1 * torch.randn(Hkv * hd, generator=gen)).to(dtype) if qknorm else None
    k_old = torch.randn(B, Hkv, past, hd, generator=gen).to(dtype)
    v_old = torch.randn(B, Hkv, past, hd, generator=gen).to(dtype)
    qr, kr, vr = _rope_ref(qkv, qw, kw, B, 1, H, Hkv, hd, past, theta, eps, Lmax)
    ref = om.attention(qr, torch.cat((k_old, kr), 2), torch.cat((v_old, vr), 2), None, dtype)
    ref = ref.transpose(1, 2).reshape(B, 1, H * hd)
    sin, cos = ops.rope_tables(hd, theta, Lmax, dev)

    def fresh():
        kc = torch.full((B, Hkv, Lmax, hd), float("nan"), dtype=dtype)  # unwritten rows must never matter
        vc = torch.full((B, Hkv, Lmax, hd), float("nan"), dtype=dtype)
        kc[:, :, :past], vc[:, :, :past] = k_old, v_old
        return kc.to(dev), vc.to(dev)

    d = lambda t: None if t is None else t.to(dev)
    ws = ops.attn_decode_workspace(B, H, hd, Lmax, dev)
    kc, vc = fresh()
    out = ops.attn_decode_fused(qkv.to(dev), d(qw), d(kw), sin, cos, kc, vc, ws, B, H, Hkv, hd, past, past + 1, eps)
    assert out is not None
    assert torch.allclose(out.cpu().float(), ref.float(), rtol=2 ** -7, atol=2 ** -7)
    assert torch.allclose(kc[:, :, past].cpu().float(), kr[:, :, 0].float(), rtol=2 ** -7, atol=2 ** -7)
    assert torch.equal(vc[:, :, past].cpu(), vr[:, :, 0])
    assert torch.isnan(kc[:, :, past + 1:].float()).all()  # nothing else written
    # same rounding points as the separate kernels; only the fp32 summation order of the softmax differs
    kc2, vc2 = fresh()
    q2 = ops.qknorm_rope_kvwrite(qkv.to(dev), d(qw), d(kw), sin, cos, kc2, vc2, B, 1, H, Hkv, hd, past, eps)
    out2 = ops.attn_decode(q2, kc2, vc2, ws, B, H, Hkv, hd, past, past + 1)
    assert torch.equal(kc2[:, :, past], kc[:, :, past])
    assert torch.allclose(out2.float(), out.float(), rtol=2 ** -8, atol=2 ** -10)
    # position from device memory, grid sized for the whole cache, padding bias
    kc3, vc3 = fresh()
    bias = torch.zeros(B, Lmax)
    if past > 8:
        bias[0, :5] = torch.finfo(torch.float32).min
    pl = torch.tensor([past], dtype=torch.int32, device=dev)
    out3 = ops.attn_decode_fused(qkv.to(dev), d(qw), d(kw), sin, cos, kc3, vc3, ws, B, H, Hkv, hd, 0, Lmax, eps,
                                 key_bias=bias.to(dev), past_len_dev=pl)
    if past > 8:
        fb = bias[:, None, None, :past + 1].to(dtype)
        fb = fb.masked_fill(fb == float("-inf"), torch.finfo(dtype).min)
        ref3 = om.attention(qr, torch.cat((k_old, kr), 2), torch.cat((v_old, vr), 2), fb, dtype)
        ref3 = ref3.transpose(1, 2).reshape(B, 1, H * hd)
        assert torch.allclose(out3.cpu().float(), ref3.float(), rtol=2 ** -7, atol=2 ** -7)
    else:
        assert torch.allclose(out3.float(), out.float(), rtol=2 ** -8, atol=2 ** -10)
    # the q and k sums of squares handed over per 16-column tile instead of being recomputed from the rows
    if qknorm:
        kc4, vc4 = fresh()
        ssq = (qkv.float() ** 2).view(B, -1, 16).sum(-1)
        out4 = ops.attn_decode_fused(qkv.to(dev), d(qw), d(kw), sin, cos, kc4, vc4, ws, B, H, Hkv, hd, past, past + 1, eps,
                                     qk_ssq=ssq.to(dev))
        assert torch.allclose(out4.float(), out.float(), rtol=2 ** -7, atol=2 ** -7)
        assert torch.allclose(kc4[:, :, past].float(), kc[:, :, past].float(), rtol=2 ** -7, atol=2 ** -7)


@pytest.mark.parametrize("merge", [0, 1, 2])
@pytest.mark.parametrize("B,past,H,Hkv,hd", [(2, 300, 4, 2, 128), (8, 2048, 32, 32, 128), (1, 1000, 8, 8, 64)])
def test_attn_decode_fused_both_merges(dev, merge, B, past, H, Hkv, hd):
    """Both ways of merging a head's key chunks (in the kernel by the last workgroup; partials + combine kernel),
    each forced on a launch the dispatcher would give to the other, against the oracle."""
    say("attn_decode_fused merge", merge, B, past, H, Hkv, hd)
    ops = _ops()
    dtype, theta, eps = torch.bfloat16, 500000.0, 1e-6
    Lmax = past + 120
    gen = torch.Generator().manual_seed(past + hd + H + merge)
    qkv = torch.randn(B, (H + 2 * Hkv) * hd, generator=gen).to(dtype)
    qw = (1 + 0.1 * torch.randn(H * hd, generator=gen)).to(dtype)
    kw = (1 + 0.1 * torch.randn(Hkv * hd, generator=gen)).to(dtype)
    k_old = torch.randn(B, Hkv, past, hd, generator=gen).to(dtype)
    v_old = torch.randn(B, Hkv, past, hd, generator=gen).to(dtype)
    qr, kr, vr = _rope_ref(qkv, qw, kw, B, 1, H, Hkv, hd, past, theta, eps, Lmax)
    ref = om.attention(qr, torch.cat((k_old, kr), 2), torch.cat((v_old, vr), 2), None, dtype)
    ref = ref.transpose(1, 2).reshape(B, 1, H * hd)
    sin, cos = ops.rope_tables(hd, theta, Lmax, dev)
    kc = torch.full((B, Hkv, Lmax, hd), float("nan"), dtype=dtype)
    vc = torch.full((B, Hkv, Lmax, hd), float("nan"), dtype=dtype)
    kc[:, :, :past], vc[:, :, :past] = k_old, v_old
    kc, vc = kc.to(dev), vc.to(dev)
    ws = ops.attn_decode_workspace(B, H, hd, Lmax, dev)
    pl = torch.tensor([past], dtype=torch.int32, device=dev)
    # twice on the same workspace: the ticket counters must be back at zero after a launch
    for rep in range(2):
        out = ops.attn_decode_fused(qkv.to(dev), qw.to(dev), kw.to(dev), sin, cos, kc, vc, ws, B, H, Hkv, hd, 0, Lmax, eps,
                                    past_len_dev=pl, merge=merge)
        assert out is not None
        assert torch.allclose(out.cpu().float(), ref.float(), rtol=2 ** -7, atol=2 ** -7), rep
    # and the dispatcher's own choice agrees with the forced one up to the order of the fp32 merge: one rounding
    # step of a bf16 output (2^-7 relative at most)
    out_auto = ops.attn_decode_fused(qkv.to(dev), qw.to(dev), kw.to(dev), sin, cos, kc, vc, ws, B, H, Hkv, hd, 0, Lmax, eps,
                                     past_len_dev=pl)
    assert torch.allclose(out_auto.float(), out.float(), rtol=2 ** -7, atol=2 ** -10)


@pytest.mark.parametrize("M", [1, 2, 4, 5, 7, 8])
@pytest.mark.parametrize("N,K,epi", [(4096, 4096, False), (12288, 4096, False), (22016, 4096, True), (768, 512, False),
                                     (4096, 11264, False), (1024, 1024, True), (4096, 11008, False), (15360, 5120, False)])
def test_w4_gemv_chain(dev, M, N, K, epi):
    """Norms chained between launches: the producer's per-tile sums of squares equal those of its output,
    and a consumer fed with them gives the same x' and y as the oracle's norm + linear (+ SwiGLU).  Up to 4 rows
    go through the kernel that keeps the activations in LDS, 5 to 8 through the one that takes them as operand
    fragments from memory."""
    say("w4_gemv_chain", M, N, K, epi)
    ops = _ops()
    gen = torch.Generator().manual_seed(M + N + K)
    a = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    resid = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    nw = (1 + 0.1 * torch.randn(K, generator=gen)).to(torch.bfloat16)
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=N + K)
    Wf = ow4.dequantize(qw, qz, sc, 128).float()
    w = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    if M <= 4 and (M + 1) * K * 2 > 128 * 1024:
        # the activations (plus a zero row) no longer fit the kernel's LDS budget: the call declines
        assert ops.w4_linear_chain(a.to(dev), w, want_ssq=not epi, swiglu_out=epi) is None
        return
    # producer side: plain product, sums of squares of its own output
    if not epi:
        r = ops.w4_linear_chain(a.to(dev), w, want_ssq=True)
        assert r is not None
        y0, _, ssq0 = r
        assert torch.equal(y0, ops.w4_linear(a.to(dev), w)) or torch.allclose(y0.float(), ops.w4_linear(a.to(dev), w).float(),
                                                                              rtol=2 ** -7, atol=2 ** -7 * y0.float().abs().max().item())
        want = (y0.float().cpu() ** 2).view(M, -1, 16).sum(-1)
        assert torch.allclose(ssq0.cpu(), want, rtol=1e-5, atol=1e-6 * want.max().item())
    # consumer side
    ssq_in = (a.float() ** 2).view(M, -1, 16).sum(-1)
    r = ops.w4_linear_chain(a.to(dev), w, resid=resid.to(dev), norm_w=nw.to(dev), eps=1e-6, ssq_in=ssq_in.to(dev),
                            swiglu_out=epi, want_ssq=not epi)
    if r is None:
        # a consumer may decline (more than 4 pieces of the row per lane); never for the 7B decode shapes
        assert K > 4096
        return
    y, x_new, ssq = r
    x_ref = resid + om.rms_norm(a, nw, 1e-6)
    y_ref = (x_ref.float() @ Wf).to(torch.bfloat16)
    if epi:
        y_ref = om.swiglu(y_ref)
    dx = (x_new.cpu().float() - x_ref.float()).abs()
    assert (dx <= 2.0 ** (torch.floor(torch.log2(x_ref.float().abs().clamp_min(1e-30))) - 7)).all()
    scale = y_ref.float().abs().max().item()
    assert (y.cpu().float() - y_ref.float()).abs().max().item() <= 2 ** -6 * scale
    if ssq is not None:
        want = (y.float().cpu() ** 2).view(M, -1, 16).sum(-1)
        assert torch.allclose(ssq.cpu(), want, rtol=1e-5, atol=1e-6 * want.max().item())


@pytest.mark.parametrize("M", [1, 8])
@pytest.mark.parametrize("N,K,epi", [
    (6144, 2048, False), (2048, 8192, False), (16384, 2048, True),       # the 1B shapes: one group per wave; K = 8192; 512 up/gate pairs
    (5120, 5120, False), (5120, 13824, False), (27648, 5120, True),      # the 13B shapes: runs of 2 or 3, of 6 or 7 and of 5 groups
    (4112, 4096, False), (24576, 4096, False), (50176, 4096, False),     # 257 tiles; 1536 tiles = 512 workgroups of three; many tiles
    (1024, 1024, False), (2048, 640, False),                            # eight groups; five (fewer than waves: the general kernel)
])
def test_w4_one_row_and_rows_kernels_over_shapes(dev, M, N, K, epi):
    """The kernels written for the decode step (one row; up to 8 rows with every request issued at once) over the
    splits of K and N their templates distinguish -- runs of equal and unequal length per wave, one and several units
    per workgroup, the slot or unit a wave or workgroup lacks asked for past the buffer -- against the oracle's norm +
    linear (+ SwiGLU); shapes they do not cover take the general kernels through the same call."""
    say("w4 one/rows shapes", M, N, K, epi)
    ops = _ops()
    gen = torch.Generator().manual_seed(M + N + K)
    a = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    resid = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    nw = (1 + 0.1 * torch.randn(K, generator=gen)).to(torch.bfloat16)
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=N + K)
    Wf = ow4.dequantize(qw, qz, sc, 128).float()
    w = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    # plain product (and the sums of squares of its output)
    y0 = ops.w4_linear(a.to(dev), w)
    y0_ref = (a.float() @ Wf).to(torch.bfloat16)
    assert (y0.cpu().float() - y0_ref.float()).abs().max().item() <= 2 ** -6 * y0_ref.float().abs().max().item()
    if not epi:
        r = ops.w4_linear_chain(a.to(dev), w, want_ssq=True)
        if r is not None:
            y1, _, ssq1 = r
            assert (y1.cpu().float() - y0_ref.float()).abs().max().item() <= 2 ** -6 * y0_ref.float().abs().max().item()
            want = (y1.float().cpu() ** 2).view(M, -1, 16).sum(-1)
            assert torch.allclose(ssq1.cpu(), want, rtol=1e-5, atol=1e-6 * want.max().item())
    # with the chained norm prologue (and the SwiGLU epilogue)
    ssq_in = (a.float() ** 2).view(M, -1, 16).sum(-1)
    r = ops.w4_linear_chain(a.to(dev), w, resid=resid.to(dev), norm_w=nw.to(dev), eps=1e-6, ssq_in=ssq_in.to(dev),
                            swiglu_out=epi, want_ssq=not epi)
    if r is None:
        assert K > 4096 or K < 1024  # a consumer may decline long or very short rows; never the model shapes at one row
        assert not (M == 1 and 1024 <= K <= 8192)
        return
    y, x_new, ssq = r
    x_ref = resid + om.rms_norm(a, nw, 1e-6)
    y_ref = (x_ref.float() @ Wf).to(torch.bfloat16)
    if epi:
        y_ref = om.swiglu(y_ref)
    dx = (x_new.cpu().float() - x_ref.float()).abs()
    assert (dx <= 2.0 ** (torch.floor(torch.log2(x_ref.float().abs().clamp_min(1e-30))) - 7)).all()
    assert (y.cpu().float() - y_ref.float()).abs().max().item() <= 2 ** -6 * y_ref.float().abs().max().item()
    if ssq is not None:
        want = (y.float().cpu() ** 2).view(M, -1, 16).sum(-1)
        assert torch.allclose(ssq.cpu(), want, rtol=1e-5, atol=1e-6 * want.max().item())


@pytest.mark.parametrize("M", [3, 8])
@pytest.mark.parametrize("N,K,epi,pro", [(12288, 4096, False, True), (4096, 4096, False, False), (22016, 4096, True, True),
                                         (4096, 11008, False, False), (2064, 640, False, True)])
def test_w4_gemv_r8_forms(dev, M, N, K, epi, pro):
    """The kernel for 5 to 8 rows in every tiling the variant entry offers (column tiles per workgroup, 8 or 16 waves):
    each against the oracle; tilings that split K over the same number of waves add the same numbers in the same
    order and must agree bit for bit."""
    say("w4_gemv_r8_forms", M, N, K, epi, pro)
    ops = _ops()
    gen = torch.Generator().manual_seed(M + N + K)
    a = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    resid = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    nw = (1 + 0.1 * torch.randn(K, generator=gen)).to(torch.bfloat16)
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=N + K)
    Wf = ow4.dequantize(qw, qz, sc, 128).float()
    w = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    x_ref = resid + om.rms_norm(a, nw, 1e-6) if pro else a
    y_ref = (x_ref.float() @ Wf).to(torch.bfloat16)
    if epi:
        y_ref = om.swiglu(y_ref)
    scale = y_ref.float().abs().max().item()
    ssq_in = (a.float() ** 2).view(M, -1, 16).sum(-1).to(dev)
    kw = dict(resid=resid.to(dev), norm_w=nw.to(dev), eps=1e-6, ssq_in=ssq_in) if pro else {}
    ran = 0
    for waves in (8, 16):
        first = None
        for nt in ((2, 4) if epi else (1, 2, 3)):
            r = ops.w4_linear_chain(a.to(dev), w, swiglu_out=epi, want_ssq=not epi, r8_form=(nt, waves), **kw)
            if r is None:  # a tiling whose registers would not fit is not built: the entry declines
                continue
            ran += 1
            y, x_new, ssq = r
            assert (y.cpu().float() - y_ref.float()).abs().max().item() <= 2 ** -6 * scale, (nt, waves)
            if pro:
                dx = (x_new.cpu().float() - x_ref.float()).abs()
                assert (dx <= 2.0 ** (torch.floor(torch.log2(x_ref.float().abs().clamp_min(1e-30))) - 7)).all()
            if ssq is not None:
                want = (y.float().cpu() ** 2).view(M, -1, 16).sum(-1)
                assert torch.allclose(ssq.cpu(), want, rtol=1e-5, atol=1e-6 * want.max().item())
            if first is None:
                first = y
            else:
                assert torch.equal(first, y), (nt, waves)
    assert ran >= (1 if K > 8192 else 2)  # a long K leaves one tiling whose requests fit the registers


# ------------------------------------------------------------------------------------------------
# act-order (desc_act) int4 layers
# ------------------------------------------------------------------------------------------------
def _act_order_case(K, N, seed):
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=seed)
    perm = torch.randperm(K, generator=torch.Generator().manual_seed(seed))
    g_idx = torch.empty(K, dtype=torch.int32)
    g_idx[perm] = (torch.arange(K) // 128).to(torch.int32)  # what GPTQ writes with desc_act (quantization/gptq.py order)
    q, z = ow4.unpack_qweight(qw), ow4.unpack_qzeros(qz)
    W = (sc.float()[g_idx.long()] * (q - z[g_idx.long()]).float()).half()  # qlinear_cuda_old.py:253-265 semantics
    return qw, qz, sc, g_idx, W


@pytest.mark.parametrize("M", [1, 7, 40, 300])
@pytest.mark.parametrize("K,N,free", [(512, 256, False), (4096, 1024, True)])
def test_qlinear_act_order(dev, M, K, N, free):
    """Non-sequential g_idx: rows sorted by group at post_init, activation columns gathered in forward."""
    say("qlinear act-order", M, K, N, free)
    from olmo_amd.qlinear import QuantLinear

    qw, qz, sc, g_idx, W = _act_order_case(K, N, seed=K + N)
    m = QuantLinear(4, 128, K, N, True, device=dev)
    m.qweight.copy_(qw), m.qzeros.copy_(qz), m.scales.copy_(sc), m.g_idx.copy_(g_idx)
    assert torch.equal(m.dequantize().cpu().view(torch.int16), W.view(torch.int16))  # table straight from the buffers
    m.post_init(free_checkpoint_buffers=free)
    assert m._perm is not None
    assert torch.equal(m.dequantize().cpu().view(torch.int16), W.view(torch.int16))  # and from the sorted, tiled copy
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(M)).to(torch.bfloat16)
    ref = ow4.linear_fp32(x, W)
    y = m(x.to(dev)).float().cpu()
    assert (y - ref).abs().max().item() <= 2 ** -7 * ref.abs().max().item()


def test_qlinear_act_order_uneven_groups_rejected(dev):
    from olmo_amd.qlinear import QuantLinear

    m = QuantLinear(4, 128, 256, 32, True, device=dev)
    g = torch.zeros(256, dtype=torch.int32)
    g[200:] = 1  # 200 rows in group 0, 56 in group 1
    m.g_idx.copy_(g)
    with pytest.raises(NotImplementedError):
        m.post_init()


def test_gather_columns(dev):
    ops = _ops()
    x = torch.randn(5, 1026, generator=torch.Generator().manual_seed(0)).to(torch.bfloat16)
    perm = torch.randperm(1026, generator=torch.Generator().manual_seed(1)).to(torch.int32)
    out = ops.gather_columns(x.to(dev), perm.to(dev)).cpu()
    assert torch.equal(out.view(torch.int16), x[:, perm.long()].view(torch.int16))


def test_measuring_probes(dev):
    """The two probes bench.py reports beside the achieved figures run and leave their sink untouched."""
    import ctypes

    from olmo_amd import _lib

    h = _lib.lib()
    src = torch.randint(-2 ** 31, 2 ** 31 - 1, (3 * 1024 * 1024 + 512,), dtype=torch.int32, device=dev)  # not a KiB multiple
    sink = torch.zeros(1024, dtype=torch.int32, device=dev)
    s = torch.cuda.current_stream().cuda_stream
    for nbytes in (1024, 2048, 70 * 1024, src.numel() * 4):
        assert h.olmo355_probe_stream_read(src.data_ptr(), nbytes, sink.data_ptr(), s) == 0
    assert h.olmo355_probe_stream_read(src.data_ptr(), 100, sink.data_ptr(), s) == 1  # less than one piece
    fl = ctypes.c_double(0.0)
    assert h.olmo355_probe_mfma_bf16(10, sink.data_ptr(), ctypes.byref(fl), s) == 0
    torch.cuda.synchronize()
    assert fl.value == 256 * 8 * 10 * 8 * 32768.0
    assert int(sink.abs().sum().item()) == 0
    poison_lds(dev)


@pytest.mark.parametrize("M,N,K", [(65, 256, 128), (300, 1024, 384), (2048, 2816, 512), (513, 22016, 256)])
def test_w4_gemm_swiglu_epilogue(dev, M, N, K):
    """int4 GEMM with SwiGLU in its epilogue == the separate GEMM then the SwiGLU kernel, bit for bit (the
    epilogue rounds up and gate to bf16 first), and both match the oracle."""
    say("w4_gemm_swiglu", M, N, K)
    ops = _ops()
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=M + N + K)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    t = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    fused, _ = ops.linear_fused(x.to(dev), t, swiglu_out=True)
    sep = ops.swiglu(ops.w4_linear(x.to(dev), t))
    assert fused.shape == (M, N // 2)
    assert torch.equal(fused, sep)
    lin = ow4.linear_fp32(x, ow4.dequantize(qw, qz, sc, 128)).to(torch.bfloat16).float()
    up, gate = lin[:, : N // 2], lin[:, N // 2:]
    ref = (torch.nn.functional.silu(gate).to(torch.bfloat16).float() * up)
    assert (fused.float().cpu() - ref).abs().max().item() <= 2 ** -6 * ref.abs().max().item()


# ------------------------------------------------------------------------------------------------
# sampling step
# ------------------------------------------------------------------------------------------------
def _reference_filter(logits_f32, temperature, top_k, top_p):
    """The kept set and its renormalised probabilities by the reference's recipe (olmo/beam_search.py:149-277:
    topk then softmax; sort descending, cumulative sum, exclusion mask shifted by one), in float64."""
    z = logits_f32.double() / temperature
    p = torch.softmax(z, -1)
    keep = torch.ones_like(p, dtype=torch.bool)
    if 0 < top_k < p.numel():
        kth = torch.topk(p, top_k).values[-1]
        keep &= p >= kth
    if top_p < 1.0:
        q = torch.where(keep, p, torch.zeros_like(p))
        q = q / q.sum()
        srt, idx = torch.sort(q, descending=True)
        cum = torch.cumsum(srt, -1)
        excl = cum >= top_p
        excl[1:] = excl[:-1].clone()
        excl[0] = False
        thr = srt[~excl][-1]
        keep &= q >= thr
    q = torch.where(keep, p, torch.zeros_like(p))
    return keep, q / q.sum()


@pytest.mark.parametrize("temperature,top_k,top_p", [(1.0, 0, 1.0), (0.7, 5, 1.0), (1.3, 0, 0.8), (1.0, 12, 0.6),
                                                      (2.0, 0, 0.0), (1.0, 1, 1.0)])
def test_sample_distribution_small_vocab(dev, temperature, top_k, top_p):
    """65536 draws from one 40-token distribution (one per row): every token lies in the reference's kept set,
    the frequencies fit its renormalised probabilities (chi-square), and the returned log-probability is the
    unfiltered log-softmax of the chosen token."""
    say("sample small", temperature, top_k, top_p)
    ops = _ops()
    n, rows = 40, 65536
    row = torch.randn(n, generator=torch.Generator().manual_seed(4)) * 2.0
    logits = row.repeat(rows, 1).to(dev)
    tok, lp = ops.sample(logits, temperature, top_k, top_p, seed=123, counter=7)
    tok, lp = tok.cpu(), lp.cpu()
    keep, q = _reference_filter(row, temperature, top_k, top_p)
    assert bool(keep[tok].all())
    assert torch.allclose(lp, torch.log_softmax(row, -1)[tok], atol=1e-5)
    obs = torch.bincount(tok, minlength=n).double()
    exp = q * rows
    m = exp > 0
    chi2 = float((((obs - exp) ** 2)[m] / exp[m]).sum())
    dof = int(m.sum()) - 1
    say("  chi2", chi2, "dof", dof)
    assert chi2 <= dof + 6.0 * (2.0 * max(dof, 1)) ** 0.5 + 1e-9
    if dof == 0:
        assert int(obs.max()) == rows and int(tok[0]) == int(row.argmax())
    # same (seed, counter) -> same draws; another counter -> other draws
    tok2, _ = ops.sample(logits, temperature, top_k, top_p, seed=123, counter=7)
    assert torch.equal(tok2.cpu(), tok)
    if dof > 0:
        cd = torch.tensor([8], dtype=torch.int32, device=dev)
        tok3, _ = ops.sample(logits, temperature, top_k, top_p, seed=123, counter_dev=cd)
        assert not torch.equal(tok3.cpu(), tok)


def test_sample_fp16_rows_equal_the_same_values_in_fp32(dev):
    """The sampler widens a row to fp32 first: fp16 logits give the draws of the same values stored as fp32."""
    ops = _ops()
    logits = (torch.randn(64, 5000, generator=torch.Generator().manual_seed(2)) * 3).half()
    th, lh = ops.sample(logits.to(dev), 0.9, 40, 0.95, seed=11, counter=2)
    tf, lf = ops.sample(logits.float().to(dev), 0.9, 40, 0.95, seed=11, counter=2)
    assert torch.equal(th, tf) and torch.equal(lh, lf) and len(set(th.tolist())) > 1


@pytest.mark.parametrize("scale,top_k,top_p", [(3.0, 50, 0.9), (3.0, 0, 0.95), (0.3, 40, 1.0), (0.3, 0, 0.5), (6.0, 20000, 0.999)])
def test_sample_large_vocab_bf16(dev, scale, top_k, top_p):
    """Vocabulary-sized bf16 rows: peaked rows are decided among the tokens near the maximum, flat ones
    (scale 0.3: every token within 2^-14 of the maximum) and very large k by the search over the whole row."""
    say("sample large", scale, top_k, top_p)
    ops = _ops()
    n, rows = 100352, 64
    logits = (torch.randn(rows, n, generator=torch.Generator().manual_seed(9)) * scale).to(torch.bfloat16)
    tok, lp = ops.sample(logits.to(dev), 1.0, top_k, top_p, seed=5, counter=3)
    tok, lp = tok.cpu(), lp.cpu()
    for r in range(0, rows, 7):
        row = logits[r].float()
        keep, q = _reference_filter(row, 1.0, top_k, top_p)
        p = torch.softmax(row.double(), -1)
        # membership up to rounding at the boundary: the kernel sums fp32 exponentials in fixed point
        assert p[tok[r]] >= p[keep].min() * (1 - 1e-4), (r, int(tok[r]))
        assert abs(float(lp[r]) - float(torch.log_softmax(row, -1)[tok[r]])) <= 1e-3
    assert len(set(tok.tolist())) > 1
