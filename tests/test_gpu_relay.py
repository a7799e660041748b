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
    """Sums of squares as tagged words: the float rounded to 20 mantissa bits, the low 4 bits = epoch & 0xf."""
    bits = v_f32.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    word = ((bits + 0x8) & 0xFFFFFFF0) | (epoch & 0xF)
    word = torch.where(word >= 2 ** 31, word - 2 ** 32, word)
    return word.to(torch.int32)


def unpair(p_i32: torch.Tensor):
    return (p_i32 & ~0xF).view(torch.float32), p_i32 & 0xF


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
    status = torch.zeros(8, dtype=torch.int32, device=dev)
    n_out = N // 2 if epi else N
    ssq_a = (a.float() ** 2).view(-1, 16).sum(-1)
    kw = dict(cfg=cfg, spin_limit=8)
    if norm:
        kw.update(resid=tag_host(resid, ep).to(dev), norm_w=nw.to(dev), eps=1e-6, ssq_in=pairs_host(ssq_a, ep).to(dev),
                  x_out=torch.zeros(K, dtype=torch.int32, device=dev))
    outs = []
    for rep in range(2):
        y = torch.zeros(n_out, dtype=torch.int32, device=dev)
        ssq = None if epi else torch.zeros(N // 16, dtype=torch.int32, device=dev)
        ok = ops.w4_relay(tag_host(a, ep).to(dev), w, y, epoch, status, swiglu=epi, ssq_out=ssq, **kw)
        if not ok:
            # a form may decline a shape (a wave's share of K beyond three quads of groups, the forced tile pair on an
            # odd tile count); the dispatcher's own choice never does for these shapes
            assert cfg != 0
            return
        outs.append((y.cpu(), None if ssq is None else ssq.cpu()))
    torch.cuda.synchronize()
    assert int(status[0].item()) == 0
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
        assert bool((tg == (ep & 0xF)).all())
        want = (yv ** 2).view(-1, 16).sum(-1)
        assert torch.allclose(val, want, rtol=2 ** -19, atol=1e-6 * want.max().item())  # 20 mantissa bits are kept
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
    status = torch.zeros(8, dtype=torch.int32, device=dev)
    y = torch.zeros(N, dtype=torch.int32, device=dev)
    stale = tag_host(a, ep - 1).to(dev)
    assert ops.w4_relay(stale, w, y, epoch, status, spin_limit=5)
    torch.cuda.synchronize()
    assert int(status[0].item()) == 1
    # one stale word in one wave's slice is enough
    status.zero_()
    one = tag_host(a, ep)
    one[1234] = tag_host(a, ep - 1)[1234]
    assert ops.w4_relay(one.to(dev), w, y, epoch, status, spin_limit=5)
    torch.cuda.synchronize()
    assert int(status[0].item()) == 1
    status.zero_()
    assert ops.w4_relay(tag_host(a, ep).to(dev), w, y, epoch, status, spin_limit=5)
    torch.cuda.synchronize()
    assert int(status[0].item()) == 0


def test_relay_tag_and_final(dev):
    ops = _ops()
    K, ep = 4096, 9
    gen = torch.Generator().manual_seed(2)
    f = torch.randn(K, generator=gen).to(torch.bfloat16)
    resid = torch.randn(K, generator=gen).to(torch.bfloat16)
    nw = (1 + 0.1 * torch.randn(K, generator=gen)).to(torch.bfloat16)
    epoch = torch.tensor([ep], dtype=torch.int32, device=dev)
    status = torch.zeros(8, dtype=torch.int32, device=dev)
    t = ops.relay_tag(f.to(dev), torch.zeros(K, dtype=torch.int32, device=dev), epoch)
    assert torch.equal(t.cpu(), tag_host(f, ep))
    assert torch.equal(ops.relay_untag(t).cpu(), f)
    ssq = pairs_host((f.float() ** 2).view(-1, 16).sum(-1), ep).to(dev)
    out = ops.relay_final(t, ssq, tag_host(resid, ep).to(dev), nw.to(dev), 1e-6, torch.zeros(K, dtype=torch.bfloat16, device=dev),
                          epoch, status, spin_limit=4)
    want = resid + om.rms_norm(f.view(1, K), nw, 1e-6).view(K)
    dx = (out.cpu().float() - want.float()).abs()
    assert (dx <= 2.0 ** (torch.floor(torch.log2(want.float().abs().clamp_min(1e-30))) - 7)).all()
    assert int(status[0].item()) == 0
    ops.relay_final(tag_host(f, ep - 1).to(dev), ssq, tag_host(resid, ep).to(dev), nw.to(dev), 1e-6, out, epoch, status, spin_limit=4)
    torch.cuda.synchronize()
    assert int(status[0].item()) == 1


def _rope_ref(qkv, qw, kw, H, Hkv, hd, past, theta, eps, n_pos):
    """q, k, v of one token as the oracle's attention block forms them (QK-norm over the full width, rotary)."""
    dq, dk = H * hd, Hkv * hd
    q, k, v = qkv[:, :dq], qkv[:, dq:dq + dk], qkv[:, dq + dk:]
    if qw is not None:
        q, k = om.rms_norm(q, qw, eps), om.rms_norm(k, kw, eps)
    q = q.view(1, 1, H, hd).transpose(1, 2)
    k = k.view(1, 1, Hkv, hd).transpose(1, 2)
    v = v.view(1, 1, Hkv, hd).transpose(1, 2)
    sin, cos = om.rope_tables(hd, theta, n_pos)
    q = om.apply_rope(q, sin[past:past + 1], cos[past:past + 1])
    k = om.apply_rope(k, sin[past:past + 1], cos[past:past + 1])
    return q, k, v


@pytest.mark.parametrize("qknorm,past,H,Hkv,hd,cap", [(True, 2048, 32, 32, 128, 2304), (True, 700, 4, 2, 128, 900), (False, 0, 2, 2, 64, 64),
                                                      (True, 127, 8, 8, 64, 128), (True, 4090, 40, 40, 128, 4100)])
def test_attn_decode_relay(dev, qknorm, past, H, Hkv, hd, cap):
    """The attention leg of the relay (tagged qkv and sums in, tagged row and hint out) == the oracle == the plain
    fused kernel on the same numbers; the new key / value row is appended; stale inputs end in a bounded give-up."""
    say("attn_decode_relay", qknorm, past, H, Hkv, hd)
    ops = _ops()
    dtype, theta, eps, ep = torch.bfloat16, 500000.0, 1e-6, 0x2B
    gen = torch.Generator().manual_seed(past + hd + H)
    width = (H + 2 * Hkv) * hd
    qkv = torch.randn(1, width, generator=gen).to(dtype)
    qw = (1 + 0.1 * torch.randn(H * hd, generator=gen)).to(dtype) if qknorm else None
    kw = (1 + 0.1 * torch.randn(Hkv * hd, generator=gen)).to(dtype) if qknorm else None
    k_old = torch.randn(1, Hkv, past, hd, generator=gen).to(dtype)
    v_old = torch.randn(1, Hkv, past, hd, generator=gen).to(dtype)
    qr, kr, vr = _rope_ref(qkv, qw, kw, H, Hkv, hd, past, theta, eps, cap)
    ref = om.attention(qr, torch.cat((k_old, kr), 2), torch.cat((v_old, vr), 2), None, dtype)
    ref = ref.transpose(1, 2).reshape(H * hd)
    sin, cos = ops.rope_tables(hd, theta, cap, dev)
    d = lambda t: None if t is None else t.to(dev)

    def fresh():
        kc = torch.full((1, Hkv, cap, hd), float("nan"), dtype=dtype)
        vc = torch.full((1, Hkv, cap, hd), float("nan"), dtype=dtype)
        kc[:, :, :past], vc[:, :, :past] = k_old, v_old
        return kc.to(dev), vc.to(dev)

    ws = ops.attn_decode_workspace(1, H, hd, cap, dev)
    epoch = torch.tensor([ep], dtype=torch.int32, device=dev)
    status = torch.zeros(8, dtype=torch.int32, device=dev)
    hint = torch.zeros(64 * 256, dtype=torch.int32, device=dev)
    pl = torch.tensor([past], dtype=torch.int32, device=dev)
    ssq = pairs_host((qkv.float() ** 2).view(-1, 16).sum(-1), ep).to(dev) if qknorm else None
    for rep in range(2):
        kc, vc = fresh()
        out = torch.zeros(H * hd, dtype=torch.int32, device=dev)
        hint.zero_()
        ok = ops.attn_decode_relay(tag_host(qkv.view(-1), ep).to(dev), d(qw), d(kw), sin, cos, kc, vc, ws, out, H, Hkv, hd, 0, cap, eps,
                                   epoch, status, past_len_dev=pl, qk_ssq=ssq, hint_out=hint, spin_limit=8)
        assert ok
        torch.cuda.synchronize()
        assert int(status[0].item()) == 0
        assert bool((ops.relay_tags(out) == (ep & 0xFFFF)).all())
        got = ops.relay_untag(out).cpu().float()
        assert torch.allclose(got, ref.float(), rtol=2 ** -7, atol=2 ** -7)
        assert torch.allclose(kc[0, :, past].cpu().float(), kr[0, :, 0].float(), rtol=2 ** -7, atol=2 ** -7)
        assert torch.equal(vc[0, :, past].cpu(), vr[0, :, 0])
        assert torch.isnan(kc[:, :, past + 1:].float()).all()
        # the hint: every copy carries the epoch once the launch has ended
        assert bool((hint.view(64, 256)[:, 0] == ep).all())
    # the same numbers through the plain fused kernel (exact per-tile sums): one bf16 rounding step apart at most
    kc2, vc2 = fresh()
    ssq_f = (qkv.float() ** 2).view(1, -1, 16).sum(-1).to(dev) if qknorm else None
    out2 = ops.attn_decode_fused(qkv.to(dev), d(qw), d(kw), sin, cos, kc2, vc2, ws, 1, H, Hkv, hd, 0, cap, eps, past_len_dev=pl,
                                 qk_ssq=ssq_f)
    assert torch.allclose(out2.view(-1).cpu().float(), got, rtol=2 ** -7, atol=2 ** -9)
    # stale qkv: the launch ends and says so
    kc3, vc3 = fresh()
    assert ops.attn_decode_relay(tag_host(qkv.view(-1), ep - 1).to(dev), d(qw), d(kw), sin, cos, kc3, vc3, ws, out, H, Hkv, hd, 0, cap,
                                 eps, epoch, status, past_len_dev=pl, qk_ssq=ssq, spin_limit=4)
    torch.cuda.synchronize()
    assert int(status[0].item()) == 1


def test_relay_decode_step_on_a_model(dev):
    """Whole decode steps of an OLMo-2-wired int4 model through the relay: the captured two-stream step gives the
    eager one-stream step's tokens and logits bit for bit (same kernels, same launch shapes), and the chained step's
    tokens; no wait gave up."""
    from olmo_amd import model as M
    from olmo_amd.config import ModelConfig
    from olmo_amd.generate import greedy_generate
    from olmo_amd.synthetic import build_random_model

    cfg = ModelConfig(d_model=1024, n_heads=8, n_layers=4, mlp_hidden_size=4096, rope=True, alibi=False, include_bias=False,
                      weight_tying=False, vocab_size=1000, embedding_size=1024, max_sequence_length=512, layer_norm_type="rms",
                      layer_norm_with_affine=True, layer_norm_eps=1e-6, attention_layer_norm=True, norm_after=True,
                      rope_theta=500000, attention_dropout=0.0, residual_dropout=0.0, embedding_dropout=0.0)
    model = build_random_model(cfg, torch.bfloat16, quantized=True, seed=3, device=dev, max_cache_len=512)
    ids = torch.randint(0, 1000, (1, 200), generator=torch.Generator().manual_seed(4)).to(dev)
    old = (M.RELAY, M.RELAY_TWO_STREAMS)
    try:
        M.RELAY = False
        t_chain, l_chain = greedy_generate(model, ids, None, 24, use_graph=True, return_logits=True)
        M.RELAY, M.RELAY_TWO_STREAMS = True, True
        t_graph, l_graph = greedy_generate(model, ids, None, 24, use_graph=True, return_logits=True)
        assert model._relay is not None and model._relay.covered
        say("relay plan", model._relay.plans)
        t_eager, l_eager = greedy_generate(model, ids, None, 24, use_graph=False, return_logits=True)
        M.RELAY_TWO_STREAMS = False
        t_one, l_one = greedy_generate(model, ids, None, 24, use_graph=True, return_logits=True)
    finally:
        M.RELAY, M.RELAY_TWO_STREAMS = old
    assert torch.equal(t_graph, t_eager) and torch.equal(l_graph, l_eager)
    assert torch.equal(t_graph, t_one) and torch.equal(l_graph, l_one)
    # against the chained step: the same arithmetic up to the order of fp32 sums and the 20-bit sums of squares
    assert (t_graph == t_chain).float().mean().item() >= 0.9
    assert (torch.softmax(l_graph.float(), -1) - torch.softmax(l_chain.float(), -1)).abs().max().item() <= 2e-2
