#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X: OLMo-2 7B, int4-g128 block Linears, bf16 activations.

  python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one batch-1 greedy decode step (embedding, 32 blocks, final norm, bf16 head, arg-max)
at KV context 2048, replayed from a captured HIP graph; ``value`` is decoded tokens/s with all
inputs resident in HBM.  The same run also reports batch-8 decode and the 1 x 2048 prefill, the
roofline of the dominant kernel (the int4 small-M linear: algorithmic bytes / HIP-event time over
a captured run of one step's 128 launches), the prefill GEMM rate, and the CPU oracle timed on
this box's host cores on a bounded sample.  Weights and tokens are synthetic (random).
Prints ONE JSON line on stdout; progress goes to stderr.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, published
MFMA_BF16_PEAK_TF = 2500.0  # MI355X dense bf16, published
W4_BYTES_PER_WEIGHT = 0.5 + 2.0 / 128 + 0.5 / 128  # nibble + fp16 scale and 4-bit zero per group of 128
# HBM bytes per launch of the int4 small-M linear, averaged over the four 7B block shapes, from two
# rocprofv3 --pmc runs of `bench.py --traffic-probe` (FETCH_SIZE, then WRITE_SIZE; KiB per dispatch), each
# scaled by what the same counter reads for a 256 MiB device copy (FETCH_SIZE reads half the bytes: factor
# 2.0; WRITE_SIZE factor 1.0).  Per shape, read: 26.29 / 8.89 / 46.97 / 23.73 MB against 26.15 / 8.72 /
# 46.85 / 23.43 MB of packed weights, scales and zeros; written: the output rows.
GEMV_TRAFFIC_BYTES_7B = 26.49e6


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def linear_shapes(cfg):
    d, dkv = cfg.d_model, cfg.effective_n_kv_heads * cfg.head_dim
    return [(d + 2 * dkv, d), (d, d), (cfg.hidden_size, d), (d, cfg.act_out_size)]  # (N, K)


def relay_compare(cfg, dev, ctx: int, steps: int) -> int:
    """Batch-1 decode of the 7B int4 model at KV context ``ctx``: the chained step against the opt-in relay
    (``olmo_amd.model.RELAY``: every hand-over between launches carried by tags in the data, launches alternating
    between two streams inside the captured step).  Same prompt, same weights; three repetitions of each form."""
    import torch

    from olmo_amd import model as M
    from olmo_amd.generate import DecodeSession, _prefill
    from olmo_amd.synthetic import build_random_model

    model = build_random_model(cfg, torch.bfloat16, quantized=True, seed=0, device=dev, max_cache_len=ctx + 4 * steps + 64,
                               free_checkpoint_buffers=True)
    ids = torch.randint(0, cfg.vocab_size, (1, ctx), generator=torch.Generator().manual_seed(0)).to(dev)

    def run(relay: bool, two: bool):
        M.RELAY, M.RELAY_TWO_STREAMS = relay, two
        _, cache, first, kb = _prefill(model, ids, None)
        sess = DecodeSession(model, cache, first, kb)
        sess.step()
        sess.step()
        sess.capture()
        toks = []
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            sess.step()
            toks.append(sess.ids.view(-1).clone())
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / steps
        model.relay_check()
        return dt * 1e3, torch.stack(toks)

    forms = {"chained": (False, False), "relay_one_stream": (True, False), "relay_two_streams": (True, True)}
    ms = {k: [] for k in forms}
    toks = {}
    try:
        for rep in range(3):
            for name, (relay, two) in forms.items():
                t, tk = run(relay, two)
                ms[name].append(t)
                toks[name] = tk
                log(f"[bench --relay] {name}: {t:.3f} ms/step")
    finally:
        M.RELAY, M.RELAY_TWO_STREAMS = False, True
    same = bool(torch.equal(toks["relay_one_stream"], toks["relay_two_streams"]))
    agree = float((toks["chained"] == toks["relay_one_stream"]).float().mean())
    out = {"workload": f"olmo2-7b int4-g128 greedy decode, batch 1, KV context {ctx}, {steps} captured steps",
           "ms_per_step": {k: min(v) for k, v in ms.items()}, "ms_per_step_all": ms,
           "relay_streams_same_tokens": same, "relay_vs_chained_token_agreement": agree,
           "relay_plan": {k: {n: hex(c) for n, c in v.items()} for k, v in getattr(model._relay, "plans", {}).items()} if model._relay else None}
    print(json.dumps(out), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--context", type=int, default=2048)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-bs8", action="store_true")
    ap.add_argument("--sweep", action="store_true",
                    help="isolated int4 linear sweep (M x shapes): prints a table on stderr and a JSON list on stdout")
    ap.add_argument("--config4", action="store_true",
                    help="BASELINE config 4 instead of the default line: OLMo-2 13B int4-g128, prefill 4 x 4096, "
                         "decode batch 16 at KV context 4096; prints one JSON object on stdout")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE: one plain copy of known size, then the four "
                         "int4 linears of a layer at one row; nothing is timed or printed")
    ap.add_argument("--probe-rows", type=int, default=1,
                    help="rows of the activations in --traffic-probe (8: the kernel for 5 to 8 rows)")
    ap.add_argument("--gemm-probe", action="store_true",
                    help="for rocprofv3 --pmc matrix-core counters: the four int4 block linears of a layer at 2048 "
                         "rows, three times each over distinct weights; nothing is timed or printed")
    ap.add_argument("--counters-probe", action="store_true",
                    help="for rocprofv3 --pmc over every kernel of the path: a 256 MiB device copy (the yardstick), one "
                         "prefill 1 x context and four eager batch-1 decode steps of the 7B int4 model; nothing is timed")
    ap.add_argument("--relay", action="store_true",
                    help="the batch-1 decode step of the 7B int4 model three ways in one run: the chained launches (the "
                         "product's path), the relay on one stream and the relay on two streams inside the captured step; "
                         "prints ms per step and whether the three gave the same tokens; one JSON object on stdout")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py: this build runs the whole model on ONE GPU; --gpus N with N > 1 is not supported.")
        return 2

    import torch

    from olmo_amd import ops
    from olmo_amd.config import PRESETS
    from olmo_amd.generate import DecodeSession, _prefill
    from olmo_amd.qlinear import QuantLinear
    from olmo_amd.synthetic import build_random_model

    if not torch.cuda.is_available():
        log("bench.py needs the GPU")
        return 2
    dev = torch.device("cuda:0")
    cfg = PRESETS["olmo2-7b"]
    if args.traffic_probe:
        return traffic_probe(cfg, dev, rows=args.probe_rows)
    if args.gemm_probe:
        return traffic_probe(cfg, dev, rows=2048)
    if args.sweep:
        return linear_sweep(dev)
    if args.config4:
        return config4(dev, args.steps if args.steps != 128 else 32)
    if args.relay:
        return relay_compare(cfg, dev, args.context, args.steps if args.steps != 128 else 64)
    ctx, K, W = args.context, args.steps, args.warmup
    cap = ctx + K + W + 8
    t0 = time.time()
    model = build_random_model(cfg, torch.bfloat16, quantized=True, seed=0, device=dev, max_cache_len=cap,
                               free_checkpoint_buffers=True)
    torch.cuda.synchronize()
    log(f"[bench] model built in {time.time() - t0:.1f}s")
    gen = torch.Generator().manual_seed(0)
    if args.counters_probe:
        src = torch.randint(0, 255, (256 << 20,), dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
        ids = torch.randint(0, cfg.vocab_size, (1, ctx), generator=gen).to(dev)
        out, cache, first, kb = _prefill(model, ids, None)
        sess = DecodeSession(model, cache, first, kb)
        for _ in range(4):
            sess.step()
        torch.cuda.synchronize()
        return 0

    def run_decode(B: int):
        ids = torch.randint(0, cfg.vocab_size, (B, ctx), generator=gen).to(dev)
        # prefill (timed separately, second run = warm; the first run's cache is given back before it, as a server
        # that finished a request would have done, so that the allocator hands the same memory out again)
        out = cache = first = kb = None
        for rep in range(2):
            out = cache = first = kb = None
            torch.cuda.synchronize()
            tp = time.perf_counter()
            out, cache, first, kb = _prefill(model, ids, None)
            torch.cuda.synchronize()
            t_prefill = time.perf_counter() - tp
        sess = DecodeSession(model, cache, first, kb)
        sess.step()
        sess.step()
        sess.capture()
        for _ in range(max(W - 2, 0)):
            sess.step()
        torch.cuda.synchronize()
        ts = time.perf_counter()
        for _ in range(K):
            sess.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - ts
        return dt, t_prefill, sess

    dt1, t_prefill, sess1 = run_decode(1)
    ms_per_step = dt1 / K * 1e3
    tok_s = K / dt1
    log(f"[bench] bs1 decode: {ms_per_step:.3f} ms/step, {tok_s:.1f} tok/s; prefill 1x{ctx}: {t_prefill * 1e3:.1f} ms")
    extra = {"prefill_tokens_per_s": ctx / t_prefill, "prefill_ms": t_prefill * 1e3}

    # ---- roofline of the dominant kernel: the int4 small-M linear --------------------------------
    # Timed: exactly the launches a decode step issues for its block Linears (olmo_amd.model.OLMo._block_decode_chain
    # without the attention launch): att_proj with the chained-norm prologue and the per-tile sums of squares,
    # attn_out, ff_proj with the chained-norm prologue and the SwiGLU epilogue, ff_out -- 128 launches over the 32
    # layers' distinct weights (3.36 GB, so neither L2 nor the 256 MB Infinity Cache can serve them), captured into
    # one graph, HIP events around its replays on the stream that replays it.
    shapes = linear_shapes(cfg)
    qls = [m for m in model.modules() if isinstance(m, QuantLinear)]
    blocks = list(model.transformer["blocks"])
    eps = cfg.layer_norm_eps
    x_res = torch.randn(1, 1, cfg.d_model, device=dev).to(torch.bfloat16)
    att_in = torch.randn(1, 1, cfg.d_model, device=dev).to(torch.bfloat16)

    def one_step_of_linears():
        x, pend = x_res, None
        for blk in blocks:
            if pend is None:
                ops.w4_linear_chain(x, blk.att_proj.tiled, want_ssq=True)
            else:
                _, x, _ = ops.w4_linear_chain(pend[0], blk.att_proj.tiled, resid=x, norm_w=pend[1], eps=eps, ssq_in=pend[2],
                                              want_ssq=True)
            a, _, ssq_a = ops.w4_linear_chain(att_in, blk.attn_out.tiled, want_ssq=True)
            u, x, _ = ops.w4_linear_chain(a, blk.ff_proj.tiled, resid=x, norm_w=blk.attn_norm.weight.data, eps=eps,
                                          ssq_in=ssq_a, swiglu_out=True)
            f, _, ssq_f = ops.w4_linear_chain(u, blk.ff_out.tiled, want_ssq=True)
            pend = (f, blk.ff_norm.weight.data, ssq_f)

    def timed_graph(fn, reps=20):
        fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / reps

    reps = 20
    n_launch = len(qls)
    avg_s = timed_graph(one_step_of_linears, reps) / n_launch
    bytes_per_launch = sum(n * k * W4_BYTES_PER_WEIGHT + 2 * k + 2 * n for n, k in shapes) * cfg.n_layers / n_launch
    achieved = bytes_per_launch / avg_s / 1e9
    roofline = {"bound": "hbm", "kernel": "w4_gemv_one_kernel (M=1): the decode step's own 4 block-Linear launches x 32 layers "
                                          "(chained-norm prologues, SwiGLU epilogue, per-tile sums of squares)",
                "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                "traffic": GEMV_TRAFFIC_BYTES_7B,
                "traffic_source": "profiles/w4_gemv_one_kernel_7b_m1_hbm_traffic.md (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE "
                                  "of `bench.py --traffic-probe`, scaled by a 256 MiB copy)",
                "avg_launch_us": avg_s * 1e6, "bytes_per_launch": bytes_per_launch}
    log(f"[bench] int4 decode linears (the step's own launches): {avg_s * 1e6:.2f} us/launch avg, {achieved:.0f} GB/s = "
        f"{achieved / HBM_PEAK_GBS:.1%} of HBM peak")

    # the same weights through plain launches (no prologue / epilogue): what the isolated kernel does
    xs = {k: torch.randn(1, k, device=dev).to(torch.bfloat16) for k in {s[1] for s in shapes}}

    def plain_linears():
        for q in qls:
            ops.w4_linear(xs[q.infeatures], q.tiled)

    plain_s = timed_graph(plain_linears, reps) / n_launch
    extra["plain_linear_launches"] = {"avg_launch_us": plain_s * 1e6, "achieved": bytes_per_launch / plain_s / 1e9, "unit": "GB/s",
                                      "frac": bytes_per_launch / plain_s / 1e9 / HBM_PEAK_GBS}
    log(f"[bench] int4 linears, plain launches: {plain_s * 1e6:.2f} us/launch = {bytes_per_launch / plain_s / 1e9:.0f} GB/s")

    # ---- prefill GEMMs (M = context): TFLOP/s against the bf16 MFMA peak ---------------------------
    # In situ: HIP events around each of the 4 x n_layers block GEMMs while a whole 1 x ctx prefill runs (norms,
    # attention and the other layers' launches between them, every layer's own weights), sum of 2MNK over the sum of
    # the kernels' times.  Beside it the same four shapes launched back to back on one layer's weights.
    ids_p = torch.randint(0, cfg.vocab_size, (1, ctx), generator=gen).to(dev)
    with ops.gemm_events() as rec:
        _prefill(model, ids_p, None)
        torch.cuda.synchronize()
    rows = [r for r in rec.rows() if r[2] == ctx]
    by_shape = {}
    for n, k, m, sec in rows:
        f, t = by_shape.get((n, k), (0.0, 0.0))
        by_shape[(n, k)] = (f + 2.0 * m * n * k, t + sec)
    situ_flops, situ_s = sum(v[0] for v in by_shape.values()), sum(v[1] for v in by_shape.values())
    tf_situ = situ_flops / situ_s / 1e12
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    xp = {k: torch.randn(ctx, k, device=dev).to(torch.bfloat16) for k in {s[1] for s in shapes}}
    layer = qls[:4]
    for q in layer:
        ops.w4_linear(xp[q.infeatures], q.tiled)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(3):
        for q in layer:
            ops.w4_linear(xp[q.infeatures], q.tiled)
    e1.record()
    torch.cuda.synchronize()
    flops = sum(2.0 * ctx * n * k for n, k in shapes)
    tf = flops * 3 / (e0.elapsed_time(e1) * 1e-3) / 1e12
    extra["prefill_gemm"] = {"bound": "mfma", "achieved": tf_situ, "peak": MFMA_BF16_PEAK_TF, "unit": "TFLOP/s",
                             "frac": tf_situ / MFMA_BF16_PEAK_TF, "M": ctx, "launches": len(rows),
                             "what": f"the block Linears' GEMM launches inside one whole 1 x {ctx} prefill of the model "
                                     "(every layer's own weights, the other kernels of the prefill between them), HIP events "
                                     "around each launch: sum of 2MNK over the sum of the launches' times",
                             "per_shape": {f"N{n}_K{k}": {"TFLOP/s": f / t / 1e12, "frac": f / t / 1e12 / MFMA_BF16_PEAK_TF,
                                                          "avg_launch_us": t / max(1, sum(1 for r in rows if r[:2] == (n, k))) * 1e6}
                                           for (n, k), (f, t) in by_shape.items()},
                             "back_to_back": {"achieved": tf, "unit": "TFLOP/s", "frac": tf / MFMA_BF16_PEAK_TF,
                                              "what": "the four block Linears of one layer at M rows through "
                                                      "olmo_amd.ops.w4_linear, three times each, HIP events around the twelve "
                                                      "launches (no SwiGLU epilogue, no other kernels between them)"}}
    log(f"[bench] int4 prefill GEMMs (M={ctx}) inside the prefill: {tf_situ:.0f} TFLOP/s = {tf_situ / MFMA_BF16_PEAK_TF:.1%} of bf16 "
        f"MFMA peak over {len(rows)} launches; back to back on one layer: {tf:.0f} TFLOP/s = {tf / MFMA_BF16_PEAK_TF:.1%}")
    for key, v in extra["prefill_gemm"]["per_shape"].items():
        log(f"[bench]   {key}: {v['TFLOP/s']:.0f} TFLOP/s = {v['frac']:.1%}, {v['avg_launch_us']:.0f} us/launch")
    # yardstick: the vendor library's *dense* bf16 GEMM (torch.matmul -> hipBLASLt) on the same four shapes at the
    # same M, nothing to dequantise: what a tuned library reaches at this size on this box
    wd = [torch.randn(n, k, device=dev).to(torch.bfloat16) * 0.02 for n, k in shapes]
    for wmat in wd:
        torch.matmul(xp[wmat.shape[1]], wmat.t())
    torch.cuda.synchronize()
    e0.record()
    for _ in range(3):
        for wmat in wd:
            torch.matmul(xp[wmat.shape[1]], wmat.t())
    e1.record()
    torch.cuda.synchronize()
    tf_lib = flops * 3 / (e0.elapsed_time(e1) * 1e-3) / 1e12
    del wd
    extra["prefill_gemm"]["vendor_library_dense_bf16_same_shapes"] = {
        "what": "torch.matmul (hipBLASLt) on dense bf16 weights of the same four shapes at the same M", "achieved": tf_lib,
        "unit": "TFLOP/s", "frac": tf_lib / MFMA_BF16_PEAK_TF}
    log(f"[bench] yardstick: vendor library, dense bf16 GEMMs of the same shapes (M={ctx}): {tf_lib:.0f} TFLOP/s = "
        f"{tf_lib / MFMA_BF16_PEAK_TF:.1%} of bf16 MFMA peak")
    # ---- the two attention kernels on their own: decode (HBM-bound) and prefill (matrix cores) -----------------
    H, hd = cfg.n_heads, cfg.head_dim
    n_lay = 16  # distinct caches, so that no launch finds its keys in a cache
    qkv1 = torch.randn(1, 3 * H * hd, device=dev).to(torch.bfloat16)
    ones = torch.ones(H * hd, device=dev).to(torch.bfloat16)
    sin_t, cos_t = ops.rope_tables(hd, float(cfg.rope_theta), cap, dev)
    kvs = [(torch.randn(1, H, cap, hd, device=dev).to(torch.bfloat16), torch.randn(1, H, cap, hd, device=dev).to(torch.bfloat16))
           for _ in range(n_lay)]
    aws = ops.attn_decode_workspace(1, H, hd, cap, dev)
    pos_dev = torch.tensor([ctx], dtype=torch.int32, device=dev)
    ssq1 = torch.rand(1, 3 * H * hd // 16, device=dev) * 16
    rope_now = torch.cat([sin_t[ctx], cos_t[ctx]]).contiguous()

    def decode_attention_launches():
        for kc_, vc_ in kvs:
            ops.attn_decode_fused(qkv1, ones, ones, sin_t, cos_t, kc_, vc_, aws, 1, H, H, hd, 0, cap, cfg.layer_norm_eps,
                                  past_len_dev=pos_dev, qk_ssq=ssq1, rope_now=rope_now)

    att_s = timed_graph(decode_attention_launches, reps) / n_lay
    att_bytes = 2.0 * (ctx + 1) * hd * 2 * H + 3 * H * hd * 2  # keys and values of every head, the token's q | k | v
    extra["decode_attention"] = {"bound": "hbm", "achieved": att_bytes / att_s / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                 "frac": att_bytes / att_s / 1e9 / HBM_PEAK_GBS, "avg_launch_us": att_s * 1e6,
                                 "what": f"attn_decode_fused_kernel (QK-norm, rotary, cache append, attention, merge), batch 1, "
                                         f"{ctx + 1} keys, {H} heads, one captured graph of {n_lay} launches over distinct caches"}
    log(f"[bench] decode attention (batch 1, {ctx + 1} keys): {att_s * 1e6:.2f} us/launch, {att_bytes / att_s / 1e9:.0f} GB/s = "
        f"{att_bytes / att_s / 1e9 / HBM_PEAK_GBS:.1%} of HBM peak")
    del kvs
    qp = torch.randn(1, ctx, H * hd, device=dev).to(torch.bfloat16)
    kp = torch.randn(1, H, ctx + 16, hd, device=dev).to(torch.bfloat16)
    vp = torch.randn(1, H, ctx + 16, hd, device=dev).to(torch.bfloat16)
    ops.attn_prefill(qp, kp, vp, 1, ctx, H, H, hd, 0)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(5):
        ops.attn_prefill(qp, kp, vp, 1, ctx, H, H, hd, 0)
    e1.record()
    torch.cuda.synchronize()
    pf_s = e0.elapsed_time(e1) * 1e-3 / 5
    pf_flops = 4.0 * H * hd * ctx * (ctx + 1) / 2
    extra["prefill_attention"] = {"bound": "mfma", "achieved": pf_flops / pf_s / 1e12, "peak": MFMA_BF16_PEAK_TF, "unit": "TFLOP/s",
                                  "frac": pf_flops / pf_s / 1e12 / MFMA_BF16_PEAK_TF, "avg_launch_us": pf_s * 1e6,
                                  "what": f"attn_prefill_mfma_kernel, 1 x {ctx} tokens, {H} heads of {hd}, causal: 4 T (T + 1) hd / 2 "
                                          "flop per head"}
    log(f"[bench] prefill attention (1 x {ctx}): {pf_s * 1e6:.1f} us, {pf_flops / pf_s / 1e12:.0f} TFLOP/s = "
        f"{pf_flops / pf_s / 1e12 / MFMA_BF16_PEAK_TF:.1%} of bf16 MFMA peak")
    del qp, kp, vp

    # ---- what this box gives a kernel that only streams the same weights / only issues MFMAs ----------
    # Same launches as the decode Linears above (one per block Linear, distinct buffers, one captured graph), but the kernel reads
    # the tiled weight bytes and does nothing else: the distance from here to the published 8 TB/s is not the
    # linear kernel's to close.  The matrix-core probe runs v_mfma_f32_16x16x32_bf16 (the GEMM's instruction) on
    # random operands.
    from olmo_amd._lib import check as _check, lib as _lib

    sink = torch.zeros(1024, dtype=torch.int32, device=dev)

    def stream_all():
        st_ = torch.cuda.current_stream().cuda_stream
        for q in qls:
            t = q.tiled
            _check("olmo355_probe_stream_read",
                   _lib().olmo355_probe_stream_read(t.wt.data_ptr(), t.wt.numel() * t.wt.element_size(), sink.data_ptr(), st_))

    stream_all()
    torch.cuda.synchronize()
    gs = torch.cuda.CUDAGraph()
    with torch.cuda.graph(gs):
        stream_all()
    gs.replay()
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        gs.replay()
    e1.record()
    torch.cuda.synchronize()
    s_avg = e0.elapsed_time(e1) * 1e-3 / (reps * n_launch)
    wt_bytes = sum(q.tiled.wt.numel() * q.tiled.wt.element_size() for q in qls) / n_launch
    assert int(sink.abs().sum().item()) == 0
    extra["ceilings"] = {
        "stream_read": {"what": "a kernel that only reads the same int4 weight tiles, same 128 launches in one graph",
                        "avg_launch_us": s_avg * 1e6, "bytes_per_launch": wt_bytes, "achieved": wt_bytes / s_avg / 1e9,
                        "unit": "GB/s", "linear_time_over_stream_time": avg_s / s_avg},
    }
    log(f"[bench] ceiling on this box: streaming the same weights {s_avg * 1e6:.2f} us/launch = {wt_bytes / s_avg / 1e9:.0f} GB/s "
        f"(linear / stream = {avg_s / s_avg:.2f})")
    # ... and all 128 weight buffers streamed by ONE launch of a persistent grid: no launch boundary, no ramp
    import ctypes as _ct

    ptrs = (_ct.c_void_p * n_launch)(*[q.tiled.wt.data_ptr() for q in qls])
    sizes = (_ct.c_int64 * n_launch)(*[q.tiled.wt.numel() * q.tiled.wt.element_size() for q in qls])

    def stream_many():
        _check("olmo355_probe_stream_read_many",
               _lib().olmo355_probe_stream_read_many(ptrs, sizes, n_launch, sink.data_ptr(), torch.cuda.current_stream().cuda_stream))

    stream_many()
    torch.cuda.synchronize()
    e0.record()
    for _ in range(5):
        stream_many()
    e1.record()
    torch.cuda.synchronize()
    m_s = e0.elapsed_time(e1) * 1e-3 / 5
    assert int(sink.abs().sum().item()) == 0
    extra["ceilings"]["stream_read_one_persistent_launch"] = {
        "what": "the same 128 weight buffers (3.3 GB) read by one launch of a grid that stays (2 workgroups per CU, 8 KiB in flight per wave at all times)",
        "ms": m_s * 1e3, "achieved": sum(sizes) / m_s / 1e9, "unit": "GB/s", "frac_of_peak": sum(sizes) / m_s / 1e9 / HBM_PEAK_GBS}
    log(f"[bench] ceiling on this box: one persistent launch streaming all weights: {m_s * 1e3:.3f} ms = {sum(sizes) / m_s / 1e9:.0f} GB/s")

    # matrix cores alone, after the GEMM timing (a sustained MFMA burst lowers the clocks of what follows)
    import ctypes

    fl = ctypes.c_double(0.0)
    _check("olmo355_probe_mfma_bf16", _lib().olmo355_probe_mfma_bf16(2000, sink.data_ptr(), ctypes.byref(fl),
                                                                     torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    e0.record()
    _check("olmo355_probe_mfma_bf16", _lib().olmo355_probe_mfma_bf16(20000, sink.data_ptr(), ctypes.byref(fl),
                                                                     torch.cuda.current_stream().cuda_stream))
    e1.record()
    torch.cuda.synchronize()
    mfma_tf = fl.value / (e0.elapsed_time(e1) * 1e-3) / 1e12
    extra["ceilings"]["mfma_bf16_random_operands"] = {"achieved": mfma_tf, "unit": "TFLOP/s",
                                                      "frac_of_peak": mfma_tf / MFMA_BF16_PEAK_TF}
    log(f"[bench] ceiling on this box: MFMA-only bf16 (16x16x32, random operands, all CUs): {mfma_tf:.0f} TFLOP/s")
    del xp

    # ---- batch 8 ------------------------------------------------------------------------------------
    if not args.no_bs8:
        del sess1
        dt8, t_prefill8, _ = run_decode(8)
        extra["decode_bs8_tokens_per_s"] = 8 * K / dt8
        extra["decode_bs8_ms_per_step"] = dt8 / K * 1e3
        extra["prefill_bs8_tokens_per_s"] = 8 * ctx / t_prefill8
        log(f"[bench] bs8 decode: {dt8 / K * 1e3:.3f} ms/step, {8 * K / dt8:.1f} tok/s")

    # ---- CPU baseline: the oracle on this box's host cores, bounded sample ------------------------------
    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(cfg, ctx)

    line = {
        "metric": "OLMo-2-7B int4 decode tok/s (bs1/bs8) + prefill tok/s; % of HBM/MFMA roofline",
        "value": tok_s, "unit": "tokens/s", "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"olmo2-7b int4-g128 greedy decode, batch 1, KV context {ctx} (+ batch 8, prefill 1x{ctx})",
                   "weights": "random int4 g128 (uniform nibbles, fp16 scales |N(0,0.01)|), bf16 head/embedding N(0,0.02)"},
        "roofline": roofline, "cpu_baseline": cpu, "extra": extra,
    }
    print(json.dumps(line), flush=True)
    return 0


def linear_sweep(dev) -> int:
    """The isolated int4 linear over M x (N, K): launches over distinct weight copies (>= 2 GB or 64 copies,
    so no cache level can serve them) timed inside a captured graph.  (The bit-exactness of the dequantised
    table for such shapes is a test, tests/test_gpu_ops.py, not part of the timing.)
    M <= 64 is reported as GB/s of algorithmic bytes against the HBM peak, M >= 512 as TFLOP/s against the
    bf16 MFMA peak."""
    import torch

    from olmo_amd import ops
    from olmo_amd.qlinear import QuantLinear
    from olmo_amd.synthetic import fill_random_int4

    gen = torch.Generator(device=dev).manual_seed(0)
    rows = []
    for n, k in [(4096, 4096), (11008, 4096), (4096, 11008), (13824, 5120), (100352, 4096)]:
        per = n * k * W4_BYTES_PER_WEIGHT
        ncopy = int(min(64, max(4, -(-2e9 // per))))
        tiles = []
        for i in range(ncopy):
            q = QuantLinear(4, 128, k, n, True, device=dev)
            fill_random_int4(q, gen)
            q.post_init(free_checkpoint_buffers=True)
            tiles.append(q.tiled)
        for m in (1, 8, 64, 512, 4096):
            x = torch.randn(m, k, device=dev).to(torch.bfloat16)

            def run():
                for t in tiles:
                    ops.w4_linear(x, t)

            run()
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                run()
            g.replay()
            torch.cuda.synchronize()
            reps = 5 if m <= 64 else 2
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                g.replay()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / (reps * ncopy)
            by = per + 2 * m * k + 2 * m * n
            fl = 2.0 * m * n * k
            row = {"M": m, "N": n, "K": k, "us": us, "copies": ncopy}
            if m <= 64:
                row.update(bound="hbm", achieved=by / us / 1e3, unit="GB/s", frac=by / us / 1e3 / HBM_PEAK_GBS)
            else:
                row.update(bound="mfma", achieved=fl / us / 1e6, unit="TFLOP/s", frac=fl / us / 1e6 / MFMA_BF16_PEAK_TF)
            rows.append(row)
            log(f"[sweep] M={m:5d} N={n:6d} K={k:5d}: {us:9.2f} us  {row['achieved']:8.1f} {row['unit']:8s} {row['frac']:6.1%}")
        del tiles
        # yardstick beside each cell: the vendor library's dense bf16 product of the same shape (torch.matmul ->
        # hipBLASLt; four times the weight bytes, nothing to dequantise), same rotation over >= 2 GB of copies
        nd = int(min(64, max(3, -(-2e9 // (2.0 * n * k)))))
        dense = [torch.randn(n, k, device=dev).to(torch.bfloat16) * 0.02 for _ in range(nd)]
        for m in (1, 8, 64, 512, 4096):
            x = torch.randn(m, k, device=dev).to(torch.bfloat16)

            def run_lib():
                for wmat in dense:
                    torch.matmul(x, wmat.t())

            run_lib()
            run_lib()
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                run_lib()
            g.replay()
            torch.cuda.synchronize()
            reps = 5 if m <= 64 else 2
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                g.replay()
            e1.record()
            torch.cuda.synchronize()
            us_lib = e0.elapsed_time(e1) * 1e3 / (reps * nd)
            for row in rows:
                if (row["M"], row["N"], row["K"]) == (m, n, k):
                    row["vendor_dense_bf16_us"] = us_lib
            log(f"[sweep] M={m:5d} N={n:6d} K={k:5d}: vendor library, dense bf16: {us_lib:9.2f} us")
        del dense
    print(json.dumps(rows))
    return 0


def config4(dev, steps: int) -> int:
    """OLMo-2 13B int4-g128 (random weights): prefill 4 x 4096 (16384 rows), then greedy decode of 16 sequences
    at KV context 4096, graph-replayed.  Algorithmic work: 415.8 TFLOP in the block GEMMs of the prefill;
    per decode step 6.59 GB of int4 weights + 1.03 GB bf16 head + 53.7 GB of KV cache."""
    import torch

    from olmo_amd.config import PRESETS
    from olmo_amd.generate import DecodeSession, _prefill
    from olmo_amd.synthetic import build_random_model

    cfg = PRESETS["olmo2-13b"]
    ctx = 4096
    model = build_random_model(cfg, torch.bfloat16, quantized=True, seed=0, device=dev, max_cache_len=ctx + steps + 16,
                               free_checkpoint_buffers=True)
    gen = torch.Generator().manual_seed(0)
    ids4 = torch.randint(0, cfg.vocab_size, (4, ctx), generator=gen).to(dev)
    for _ in range(2):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        _prefill(model, ids4, None)
        torch.cuda.synchronize()
        t_prefill = time.perf_counter() - t0
    d, h, L = cfg.d_model, cfg.hidden_size, cfg.n_layers
    gemm_flop = 2.0 * 4 * ctx * L * (d * 3 * d + d * d + d * h + (h // 2) * d)
    log(f"[config4] prefill 4x{ctx}: {t_prefill * 1e3:.1f} ms = {4 * ctx / t_prefill:.0f} tok/s "
        f"({gemm_flop / t_prefill / 1e12:.0f} TFLOP/s counting the block GEMMs only)")
    ids16 = torch.randint(0, cfg.vocab_size, (16, ctx), generator=gen).to(dev)
    out, cache, first, kb = _prefill(model, ids16, None)
    sess = DecodeSession(model, cache, first, kb)
    sess.step()
    sess.step()
    sess.capture()
    for _ in range(4):
        sess.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        sess.step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    kv_bytes = 2.0 * 16 * L * cfg.effective_n_kv_heads * cfg.head_dim * 2 * (ctx + 6 + steps / 2)
    w_bytes = L * (d * 3 * d + d * d + d * h + (h // 2) * d) * W4_BYTES_PER_WEIGHT + 2.0 * d * cfg.logits_size
    log(f"[config4] decode batch 16 at context {ctx}: {dt * 1e3:.2f} ms/step = {16 / dt:.0f} tok/s; "
        f"{(kv_bytes + w_bytes) / dt / 1e9:.0f} GB/s of KV cache + weights")
    print(json.dumps({"workload": "olmo2-13b int4-g128: prefill 4x4096, decode batch 16 at KV context 4096",
                      "prefill_ms": t_prefill * 1e3, "prefill_tokens_per_s": 4 * ctx / t_prefill,
                      "prefill_block_gemm_tflops": gemm_flop / t_prefill / 1e12,
                      "decode_ms_per_step": dt * 1e3, "decode_tokens_per_s": 16 / dt,
                      "decode_bytes_per_step": kv_bytes + w_bytes, "decode_gbs": (kv_bytes + w_bytes) / dt / 1e9,
                      "steps": steps}), flush=True)
    return 0


def traffic_probe(cfg, dev, rows: int = 1) -> int:
    """Launches whose hardware counters are read: a 256 MiB device copy (the yardstick for HBM traffic: 256 MiB
    read, 256 MiB written) and the four int4 block linears at ``rows`` rows, three times each over distinct
    weights."""
    import torch

    from olmo_amd import ops
    from olmo_amd.qlinear import QuantLinear
    from olmo_amd.synthetic import fill_random_int4

    gen = torch.Generator(device=dev).manual_seed(0)
    src = torch.randint(0, 255, (256 << 20,), dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    dst.copy_(src)
    torch.cuda.synchronize()
    for n, k in linear_shapes(cfg):
        x = torch.randn(rows, k, device=dev).to(torch.bfloat16)
        for _ in range(3):
            q = QuantLinear(4, 128, k, n, True, device=dev)
            fill_random_int4(q, gen)
            q.post_init(free_checkpoint_buffers=True)
            torch.cuda.synchronize()
            ops.w4_linear(x, q.tiled)
            torch.cuda.synchronize()
            del q
    return 0


def cpu_baseline(cfg, ctx: int):
    """Oracle (pure torch on the CPU, dequantise-then-matmul per call as the reference's QuantLinear
    does) on a bounded sample: 2 of the 32 layers of the same 7B int4 shape, 2 decode steps at KV
    context ``ctx`` with a random cache; scaled to 32 layers + head."""
    import copy

    import torch

    from oracle import model as om

    n_sample = 2
    c2 = copy.copy(cfg)
    c2.n_layers = n_sample
    c2.embedding_size = 1024  # the sample skips the 0.8 GB head; its time is added from a separate timing
    c2.vocab_size = 1000
    t0 = time.time()
    w = om.random_weights(c2, torch.bfloat16, seed=1, quantized=True)
    oracle = om.OracleModel(c2, w, torch.bfloat16, cache_weights=False)
    hd, H = cfg.head_dim, cfg.n_heads
    kv = [(torch.randn(1, H, ctx, hd).bfloat16(), torch.randn(1, H, ctx, hd).bfloat16()) for _ in range(n_sample)]
    ids = torch.randint(0, 1000, (1, 1))
    log(f"[bench] cpu baseline: sample built in {time.time() - t0:.1f}s, threads={torch.get_num_threads()}")
    times = []
    for _ in range(2):
        ts = time.perf_counter()
        oracle.forward(ids, past_key_values=kv, use_cache=True, last_logits_only=True)
        times.append(time.perf_counter() - ts)
    per_layer = min(times) / n_sample
    head = torch.randn(cfg.logits_size, cfg.d_model).bfloat16()
    x = torch.randn(1, cfg.d_model).bfloat16()
    ts = time.perf_counter()
    (x.float() @ head.float().t()).bfloat16()
    t_head = time.perf_counter() - ts
    t_token = per_layer * cfg.n_layers + t_head
    log(f"[bench] cpu baseline: {per_layer:.2f} s/layer, head {t_head:.2f} s -> {1.0 / t_token:.4f} tok/s")
    # BASELINE configs[0] in full (the reference's own CPU-runnable case): 20M-style fp32 model, batch 4 x 512
    from olmo_amd.config import PRESETS

    c1 = PRESETS["olmo-20m"]
    o1 = om.OracleModel(c1, om.random_weights(c1, torch.float32, seed=2), torch.float32)
    ids1 = torch.randint(0, 50280, (4, 512), generator=torch.Generator().manual_seed(3))
    t_c1 = []
    for _ in range(2):
        ts = time.perf_counter()
        o1.forward(ids1)
        t_c1.append(time.perf_counter() - ts)
    log(f"[bench] cpu baseline: 20M fp32 model, forward on 4 x 512 tokens: {min(t_c1):.2f} s = {2048 / min(t_c1):.0f} tok/s")
    return {"value": 1.0 / t_token, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{n_sample} of {cfg.n_layers} layers x 2 decode steps (best) at KV context {ctx}, batch 1, "
                      f"dequantise per call; scaled to {cfg.n_layers} layers + the bf16 head",
            "os_cpu_count": os.cpu_count(),
            "config1_20m_fp32_forward_4x512": {"seconds": min(t_c1), "tokens_per_s": 2048 / min(t_c1), "sample": "in full, best of 2"}}


if __name__ == "__main__":
    sys.exit(main())
