"""The decode relay (olmo_amd/csrc/relay.hip): int4 linears, attention and the final update with epoch-tagged
hand-overs, against the CPU oracle on the same seeded inputs, through the C-ABI; the bounded wait forced from the
host; the two-stream captured step against the one-stream eager step."""
import pytest
import torch

from oracle import model as om
from oracle import w4 as ow4

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from olmo_amd import _lib

    _lib.lib()
    return torch.device("cuda:0")


def _ops():
    from olmo_amd import ops

    return ops


def say(*a):
    print(*a, flush=True)


def tag_host(x_bf16: torch.Tensor, epoch: int) -> torch.Tensor:
    """bf16 numbers -> tagged int32 words, on the host (independent of the device's relay_tag)."""
    bits = x_bf16.contiguous().view(torch.int16).to(torch.int32) & 0xFFFF
    word = (bits.to(torch.int64) << 16) | (epoch & 0xFFFF)
    word = torch.where(word >= 2 ** 31, word - 2 ** 32, word)
    return word.to(torch.int32)


def pairs_host(v_f32: torch.Tensor, epoch: int) -> torch.Tensor:
    bits = v_f32.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    return bits | (epoch << 32)


def unpair(p_i64: torch.Tensor):
    lo = (p_i64 & 0xFFFFFFFF)
    lo = torch.where(lo >= 2 ** 31, lo - 2 ** 32, lo).to(torch.int32)
    return lo.view(torch.float32), (p_i64 >> 32) & 0xFFFFFFFF


# cfg = waves | nt << 8; 0 = the dispatcher's choice
@pytest.mark.parametrize("cfg", [0, 4 | 1 << 8, 8 | 1 << 8, 16 | 1 << 8, 8 | 2 << 8, 16 | 2 << 8])
@pytest.mark.parametrize("N,K,norm,epi", [(4096, 4096, False, False), (12288, 4096, True, False), (22016, 4096, True, True),
                                          (4096, 11008, False, False), (768, 512, True, False), (1024, 1024, True, True),
                                          (15360, 5120, True, False), (5120, 13824, False, False), (272, 1408, False, False)])
def test_w4_relay_linear(dev, N, K, norm, epi, cfg):
    """y = x' . W with x' = x or resid + rmsnorm(x) from tagged inputs == the oracle; every output word, every
    sum-of-squares pair and the residual row carry the epoch; bit-reproducible."""
    say("w4_relay", N, K, norm, epi, hex(cfg))
    ops = _ops()
    gen = torch.Generator().manual_seed(N + K)
    a = torch.randn(K, generator=gen).to(torch.bfloat16)
    resid = torch.randn(K, generator=gen).to(torch.bfloat16)
    nw = (1 + 0.1 * torch.randn(K, generator=gen)).to(torch.bfloat16)
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=N + K)
    Wf = ow4.dequantize(qw, qz, sc, 128).float()
    w = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    ep = 0x12345
    epoch = torch.tensor([ep], dtype=torch.int32, device=dev)
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    n_out = N // 2 if epi else N
    ssq_a = (a.float() ** 2).view(-1, 16).sum(-1)
    kw = dict(cfg=cfg, spin_limit=8)
    if norm:
        kw.update(resid=tag_host(resid, ep).to(dev), norm_w=nw.to(dev), eps=1e-6, ssq_in=pairs_host(ssq_a, ep).to(dev),
                  x_out=torch.zeros(K, dtype=torch.int32, device=dev))
    outs = []
    for rep in range(2):
        y = torch.zeros(n_out, dtype=torch.int32, device=dev)
        ssq = None if epi else torch.zeros(N // 16, dtype=torch.int64, device=dev)
        ok = ops.w4_relay(tag_host(a, ep).to(dev), w, y, epoch, status, swiglu=epi, ssq_out=ssq, **kw)
        if not ok:
            # a form may decline a shape (a wave's share of K beyond three quads of groups, the forced tile pair on an
            # odd tile count); the dispatcher's own choice never does for these shapes
            assert cfg != 0
            return
        outs.append((y.cpu(), None if ssq is None else ssq.cpu()))
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    assert torch.equal(outs[0][0], outs[1][0]), "not deterministic"
    y, ssq = outs[0]
    assert bool((ops.relay_tags(y) == (ep & 0xFFFF)).all())
    yv = ops.relay_untag(y).float()
    x_ref = (resid + om.rms_norm(a.view(1, K), nw, 1e-6).view(K)) if norm else a
    y_ref = (x_ref.float().view(1, K) @ Wf).to(torch.bfloat16)
    if epi:
        y_ref = om.swiglu(y_ref)
    y_ref = y_ref.view(-1).float()
    # bf16 output rounding + fp32 accumulation order: 2^-6 of the row scale, as for the one-stream kernels
    assert (yv - y_ref).abs().max().item() <= 2 ** -6 * y_ref.abs().max().item()
    if ssq is not None:
        val, tg = unpair(ssq)
        assert bool((tg == ep).all())
        want = (yv ** 2).view(-1, 16).sum(-1)
        assert torch.allclose(val, want, rtol=1e-5, atol=1e-6 * want.max().item())
    if norm:
        xo = kw["x_out"].cpu()
        assert bool((ops.relay_tags(xo) == (ep & 0xFFFF)).all())
        dx = (ops.relay_untag(xo).float() - x_ref.float()).abs()
        assert (dx <= 2.0 ** (torch.floor(torch.log2(x_ref.float().abs().clamp_min(1e-30))) - 7)).all()
    # a bf16 row in, a bf16 row out: the same numbers
    if not norm:
        y2 = torch.zeros(n_out, dtype=torch.bfloat16, device=dev)
        assert ops.w4_relay(a.to(dev), w, y2, epoch, status, cfg=cfg)
        assert torch.equal(y2.cpu(), ops.relay_untag(y))


def test_w4_relay_wait_is_bounded(dev):
    """Inputs that never show the epoch (the producer 'died'): the launch ends after spin_limit polls and says so in
    the status word; nothing hangs.  Then the same launch with good inputs leaves the status alone."""
    ops = _ops()
    N, K, ep = 4096, 4096, 77
    gen = torch.Generator().manual_seed(1)
    a = torch.randn(K, generator=gen).to(torch.bfloat16)
    qw, qz, sc = ow4.random_quantized(K, N, 128, seed=3)
    w = ops.w4_repack(qw.to(dev), qz.to(dev), sc.to(dev), 128)
    epoch = torch.tensor([ep], dtype=torch.int32, device=dev)
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    y = torch.zeros(N, dtype=torch.int32, device=dev)
    stale = tag_host(a, ep - 1).to(dev)
    assert ops.w4_relay(stale, w, y, epoch, status, spin_limit=5)
    torch.cuda.synchronize()
    assert int(status.item()) == 1
    # one stale word in one wave's slice is enough
    status.zero_()
    one = tag_host(a, ep)
    one[1234] = tag_host(a, ep - 1)[1234]
    assert ops.w4_relay(one.to(dev), w, y, epoch, status, spin_limit=5)
    torch.cuda.synchronize()
    assert int(status.item()) == 1
    status.zero_()
    assert ops.w4_relay(tag_host(a, ep).to(dev), w, y, epoch, status, spin_limit=5)
    torch.cuda.synchronize()
    assert int(status.item()) == 0


def test_relay_tag_and_final(dev):
    ops = _ops()
    K, ep = 4096, 9
    gen = torch.Generator().manual_seed(2)
    f = torch.randn(K, generator=gen).to(torch.bfloat16)
    resid = torch.randn(K, generator=gen).to(torch.bfloat16)
    nw = (1 + 0.1 * torch.randn(K, generator=gen)).to(torch.bfloat16)
    epoch = torch.tensor([ep], dtype=torch.int32, device=dev)
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    t = ops.relay_tag(f.to(dev), torch.zeros(K, dtype=torch.int32, device=dev), epoch)
    assert torch.equal(t.cpu(), tag_host(f, ep))
    assert torch.equal(ops.relay_untag(t).cpu(), f)
    ssq = pairs_host((f.float() ** 2).view(-1, 16).sum(-1), ep).to(dev)
    out = ops.relay_final(t, ssq, tag_host(resid, ep).to(dev), nw.to(dev), 1e-6, torch.zeros(K, dtype=torch.bfloat16, device=dev),
                          epoch, status, spin_limit=4)
    want = resid + om.rms_norm(f.view(1, K), nw, 1e-6).view(K)
    dx = (out.cpu().float() - want.float()).abs()
    assert (dx <= 2.0 ** (torch.floor(torch.log2(want.float().abs().clamp_min(1e-30))) - 7)).all()
    assert int(status.item()) == 0
    ops.relay_final(tag_host(f, ep - 1).to(dev), ssq, tag_host(resid, ep).to(dev), nw.to(dev), 1e-6, out, epoch, status, spin_limit=4)
    torch.cuda.synchronize()
    assert int(status.item()) == 1
