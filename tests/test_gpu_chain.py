"""The persistent chain of decode-step int4 linears (``olmo355_w4_chain``) against the oracle: single phases of
every kind, the four-phase chain of the 7B block (attn_out -> ff_proj + SwiGLU -> ff_out -> next att_proj with the
two post-norm residual updates), shapes with fewer tiles than workgroups, rotated tile ownership, repeated launches
on the same barrier counters, and a wait forced to give up from the host."""
import pytest
import torch

from oracle import model as om
from oracle import w4 as ow4

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available()
    from olmo_amd import _lib

    _lib.lib()
    return torch.device("cuda:0")


def _weight(dev, N, K, seed):
    from olmo_amd import ops

    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=seed)
    Wf = ow4.dequantize(qw, qz, sc, 128).float()
    return ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128), Wf


def _sync(dev):
    from olmo_amd import ops

    return ops.chain_sync(dev)


def _ulp_close(a, b):
    """bf16 tensors equal up to one unit in the last place of the larger magnitude."""
    a, b = a.float(), b.float()
    ulp = 2.0 ** (torch.floor(torch.log2(torch.maximum(a.abs(), b.abs()).clamp_min(1e-30))) - 7)
    return bool(((a - b).abs() <= ulp).all())


@pytest.mark.parametrize("M", [1, 3, 4])
@pytest.mark.parametrize("N,K,rot", [(4096, 4096, 0), (12288, 4096, 17), (4096, 11008, 255), (768, 512, 0), (272, 1408, 250),
                                     (16, 128, 3), (5120, 5120, 1)])
def test_single_plain_phase(dev, M, N, K, rot):
    say("chain plain", M, N, K, rot)
    from olmo_amd import ops

    w, Wf = _weight(dev, N, K, N + K)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(M)).to(torch.bfloat16)
    ref = x.float() @ Wf
    y = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    ssq = torch.full((M, N // 16), float("nan"), dtype=torch.float32, device=dev)
    sync, status = _sync(dev)
    assert ops.w4_chain([ops.ChainStep(x.to(dev), w, y, ssq_out=ssq, rot=rot % ops.chain_grid())], sync, status)
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    scale = ref.abs().max().item()
    assert (y.float().cpu() - ref).abs().max().item() <= 2 ** -7 * scale
    want = (y.float() ** 2).view(M, -1, 16).sum(-1)
    assert torch.allclose(ssq, want, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("M", [1, 2, 4])
@pytest.mark.parametrize("N,K,epi", [(22016, 4096, True), (12288, 4096, False), (1024, 1024, True), (27648, 5120, True)])
def test_single_chained_phase(dev, M, N, K, epi):
    """x' = resid + rmsnorm(a) from the producer's per-tile sums of squares, product, optional SwiGLU."""
    say("chain normed", M, N, K, epi)
    from olmo_amd import ops

    w, Wf = _weight(dev, N, K, N + K + 1)
    g = torch.Generator().manual_seed(M + N)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    resid = torch.randn(M, K, generator=g).to(torch.bfloat16)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).to(torch.bfloat16)
    x_ref = resid + om.rms_norm(a, nw, 1e-6)
    y_ref = (x_ref.float() @ Wf).to(torch.bfloat16)
    if epi:
        y_ref = om.swiglu(y_ref)
    ssq_in = (a.float() ** 2).view(M, -1, 16).sum(-1).to(dev)
    y = torch.full((M, N // 2 if epi else N), float("nan"), dtype=torch.bfloat16, device=dev)
    x_out = torch.full((M, K), float("nan"), dtype=torch.bfloat16, device=dev)
    sync, status = _sync(dev)
    step = ops.ChainStep(a.to(dev), w, y, resid=resid.to(dev), norm_w=nw.to(dev), ssq_in=ssq_in, x_out=x_out, swiglu=epi,
                         eps=1e-6, rot=5)
    assert ops.w4_chain([step], sync, status)
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    assert _ulp_close(x_out.cpu(), x_ref)
    scale = y_ref.float().abs().max().item()
    assert (y.float().cpu() - y_ref.float()).abs().max().item() <= 2 ** -6 * scale


@pytest.mark.parametrize("M", [1, 4])
@pytest.mark.parametrize("d,ff", [(4096, 11008), (512, 1024), (5120, 13824)])
def test_four_phase_block_chain(dev, M, d, ff):
    """attn_out -> [x1 = x0 + norm(a)] ff_proj + SwiGLU -> ff_out -> [x2 = x1 + norm(f)] next att_proj, launched twice
    on the same counters, against the oracle's composition (olmo/model.py:786-821) and the separate launches."""
    say("chain block", M, d, ff)
    from olmo_amd import ops

    w_o, W_o = _weight(dev, d, d, 1)
    w_up, W_up = _weight(dev, 2 * ff, d, 2)
    w_dn, W_dn = _weight(dev, d, ff, 3)
    w_qkv, W_qkv = _weight(dev, 3 * d, d, 4)
    g = torch.Generator().manual_seed(M + d)
    att = torch.randn(M, d, generator=g).to(torch.bfloat16)
    x0 = torch.randn(M, d, generator=g).to(torch.bfloat16)
    nw1 = (1 + 0.1 * torch.randn(d, generator=g)).to(torch.bfloat16)
    nw2 = (1 + 0.1 * torch.randn(d, generator=g)).to(torch.bfloat16)
    # oracle
    a = (att.float() @ W_o).to(torch.bfloat16)
    x1 = x0 + om.rms_norm(a, nw1, 1e-6)
    u = om.swiglu((x1.float() @ W_up).to(torch.bfloat16))
    f = (u.float() @ W_dn).to(torch.bfloat16)
    x2 = x1 + om.rms_norm(f, nw2, 1e-6)
    qkv = (x2.float() @ W_qkv).to(torch.bfloat16)

    def buf(*shape, dtype=torch.bfloat16):
        return torch.full(shape, float("nan"), dtype=dtype, device=dev)

    A, U, Fo, QKV, X1, X2 = buf(M, d), buf(M, ff), buf(M, d), buf(M, 3 * d), buf(M, d), buf(M, d)
    sa, sf, sq = buf(M, d // 16, dtype=torch.float32), buf(M, d // 16, dtype=torch.float32), buf(M, 3 * d // 16, dtype=torch.float32)
    attd, x0d, n1, n2 = att.to(dev), x0.to(dev), nw1.to(dev), nw2.to(dev)
    steps = [
        ops.ChainStep(attd, w_o, A, ssq_out=sa, rot=0),
        ops.ChainStep(A, w_up, U, resid=x0d, norm_w=n1, ssq_in=sa, x_out=X1, swiglu=True, eps=1e-6, rot=40),
        ops.ChainStep(U, w_dn, Fo, ssq_out=sf, rot=0),
        ops.ChainStep(Fo, w_qkv, QKV, resid=X1, norm_w=n2, ssq_in=sf, x_out=X2, ssq_out=sq, eps=1e-6, rot=7),
    ]
    sync, status = _sync(dev)
    for rep in range(2):
        for t in (A, U, Fo, QKV, X1, X2):
            t.fill_(float("nan"))
        ok = ops.w4_chain(steps, sync, status)
        if not ok:  # declined, nothing launched: the rows of the longest K (+ one weight slot per wave) exceed a CU's LDS
            assert M * ((ff + 511) // 512) * 1024 > 64 * 1024
            pytest.skip("activations of this shape do not fit next to the weight slots: the caller uses separate launches")
        torch.cuda.synchronize()
        assert int(status.item()) == 0, rep
        for name, got, ref in (("a", A, a), ("u", U, u), ("f", Fo, f), ("qkv", QKV, qkv)):
            scale = ref.float().abs().max().item()
            err = (got.float().cpu() - ref.float()).abs().max().item()
            assert err <= 2 ** -5 * scale, (rep, name, err, scale)
        for name, got, ref in (("x1", X1, x1), ("x2", X2, x2)):
            err = (got.float().cpu() - ref.float()).abs().max().item()
            assert err <= 2 ** -5 * ref.float().abs().max().item(), (rep, name, err)
    # the same steps as separate launches of the existing kernels: equal up to the order of the fp32 sums
    r1 = ops.w4_linear_chain(attd, w_o, want_ssq=True)
    r2 = ops.w4_linear_chain(r1[0], w_up, resid=x0d, norm_w=n1, eps=1e-6, ssq_in=r1[2], swiglu_out=True)
    r3 = ops.w4_linear_chain(r2[0], w_dn, want_ssq=True)
    if r1 is not None and r2 is not None and r3 is not None:
        assert (A.float() - r1[0].float()).abs().max().item() <= 2 ** -6 * a.float().abs().max().item()
        assert (Fo.float() - r3[0].float()).abs().max().item() <= 2 ** -5 * f.float().abs().max().item()
    assert torch.allclose(sq, (QKV.float() ** 2).view(M, -1, 16).sum(-1), rtol=1e-5, atol=1e-6)


def test_wait_that_gives_up_ends_the_launch(dev):
    """A spin limit of one poll forced from the host: the launch must still end, report through the status word (if
    any wait really gave up) and leave the barrier counters at zero for the next launch, which then is correct."""
    say("chain give-up")
    from olmo_amd import ops

    d = 1024
    w1, W1 = _weight(dev, d, d, 11)
    w2, W2 = _weight(dev, d, d, 12)
    x = torch.randn(2, d, generator=torch.Generator().manual_seed(0)).to(torch.bfloat16).to(dev)
    y1 = torch.zeros(2, d, dtype=torch.bfloat16, device=dev)
    y2 = torch.zeros(2, d, dtype=torch.bfloat16, device=dev)
    sync, status = _sync(dev)
    steps = [ops.ChainStep(x, w1, y1), ops.ChainStep(y1, w2, y2)]
    assert ops.w4_chain(steps, sync, status, spin_limit=1)
    torch.cuda.synchronize()
    assert int(status.item()) in (0, 1)
    status.zero_()
    assert ops.w4_chain(steps, sync, status)
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    ref1 = (x.float().cpu() @ W1).to(torch.bfloat16)
    ref2 = ref1.float() @ W2
    assert (y2.float().cpu() - ref2).abs().max().item() <= 2 ** -5 * ref2.abs().max().item()
