#!/usr/bin/env python3
"""Benchmark of the MI355X backward path.  Prints ONE JSON line.

Default workload ("linear_i8_bwd") = the int8 linear-layer backward of the reference's operator TMatMulBuffers
(BackpropMulti + Backprop + BackpropDelta): X i8 [16384x1024] with per-row scales, dY bf16 [16384x4096], W i8 [4096x1024] with
per-output-channel scales; one step = quantise dY per row, transpose W, dX GEMM, re-quantise dY per k-tile + transpose,
transpose X, delta GEMM with the packed-delta epilogue.  All inputs are resident in HBM before the timed region.

python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

PEAK_INT8 = 5.0e15   # MI355X dense int8 MFMA, op/s
PEAK_FP8 = 5.0e15
PEAK_BF16 = 2.5e15
PEAK_HBM = 8.0e12


def event_time_ms(fn, iters):
    import torch
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def sustained(ab_type):
    """What the device sustains with nothing else running: an MFMA-only kernel with per-lane random operand bits (the chip is power
    limited below its boost clock under such data) and a streaming copy.  Reported beside the published peaks, never instead of them."""
    from tscale2_amd import lib as L
    return {"mfma_only_random_operands_tops": round(L.probe_mfma_rate(ab_type, 1, 100000), 1),
            "mfma_only_constant_operands_tops": round(L.probe_mfma_rate(ab_type, 0, 100000), 1),
            "copy_read_plus_write_gbps": round(L.probe_copy_rate(1 << 30), 1)}


def cpu_baseline_linear(len_full, src_dim, grad_dim, sample_rows):
    """The oracle's restatement of the reference CPU path (MulBackwardWithAccum + SumRankOne, cpu_util.cpp:30-67), OpenMP over
    independent output rows, on a row subsample; tokens/s = sample_rows / time."""
    import numpy as np
    from oracle_lib import Oracle
    orc = Oracle()
    cores = len(os.sched_getaffinity(0))
    cores = min(cores, 16)
    os.environ["OMP_NUM_THREADS"] = str(cores)
    r = np.random.default_rng(0)
    w = (r.standard_normal((grad_dim, src_dim)) * 0.02).astype(np.float32)
    x = r.standard_normal((sample_rows, src_dim)).astype(np.float32)
    dy = r.standard_normal((sample_rows, grad_dim)).astype(np.float32)
    t0 = time.perf_counter()
    orc.mul_backward_accum(np.zeros((sample_rows, src_dim), np.float32), w, dy)
    orc.sum_rank_one(x, dy)
    dt = time.perf_counter() - t0
    return {"value": sample_rows / dt, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"{sample_rows} of {len_full} rows (dX + delta, fp32 scalar loops of the reference CPU path, OpenMP over output rows), {dt:.1f} s"}


def bench_linear_i8(args):
    import numpy as np
    import torch
    from tscale2_amd import lib as L
    L.load()
    len_, src_dim, grad_dim, k_tile = 16384, 1024, 4096, 512
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn((len_, src_dim), device="cuda", generator=g)
    dy = torch.randn((len_, grad_dim), device="cuda", generator=g)
    w = torch.randn((grad_dim, src_dim), device="cuda", generator=g) * 0.02
    # X: int8 with per-row abs-max scales; W: int8 with per-output-channel abs-max scales; dY arrives in bf16
    x_scale = x.abs().amax(dim=1) / 127
    x8 = torch.clamp(torch.round(x / x_scale[:, None]), -128, 127).to(torch.int8)
    w_scale = w.abs().amax(dim=1) / 127
    w8 = torch.clamp(torch.round(w / w_scale[:, None]), -128, 127).to(torch.int8)
    dy16 = dy.bfloat16()
    # the 4096 x 1024 delta has too few tiles for 256 CUs: two stored slices of the token axis on 256x128 tiles, packed from their sum
    splits = args.delta_splits
    bufs = L.MatMulBuffers(L.I8, len_, src_dim, grad_dim, k_tile=k_tile, splits=splits, share_row_max=True)
    dx = torch.empty((len_, src_dim), dtype=torch.float32, device="cuda")
    dyv = dy16.view(torch.int16)

    def step():
        # dX = (dY * s_w) W8 : the column scale of W lies on the contraction axis, so it is folded into dY before row quantisation
        bufs.backprop_multi(len_, w8, dyv, L.BF16, w_scale)
        bufs.backprop(len_, None, 1.0, None, dx, L.F32)
        # delta = sum_t (s_x[t] dY[t]) X8[t] : the row scale of X is folded into dY before k-tile quantisation
        bufs.backprop_delta(len_, x8, x_scale, dyv, L.BF16)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3

    # sanity of the result (not timed): against fp64 on a slice
    ref_dx = (dy16[:256].double() * w_scale.double()[None, :]) @ w8.double()
    err = ((dx[:256].double() - ref_dx).abs().max() / ref_dx.abs().max()).item()
    assert err < 3e-2, f"dX deviates from the fp64 product: {err}"

    # dominant kernel, timed alone with events on the launch stream: the two int8 MFMA GEMMs (dX and delta), 137.44 GOP each
    gemm_ops = 2.0 * len_ * src_dim * grad_dim
    ms_dx = event_time_ms(lambda: bufs.backprop(len_, None, 1.0, None, dx, L.F32), 20)
    tsc, gt, st = bufs.t["tileScale"], bufs.t["gradT"], bufs.t["srcT"]
    lib = L.load()

    def dw():
        if splits > 1:
            part = bufs.t["partial"]
            lib.gemm_nt(gt, st, part, L.I8, L.F32, k_tile_scale=tsc, k_tile=k_tile, split_k=splits, split_slab_bytes=grad_dim * src_dim * 4,
                        tile_config=3 | 8, m=grad_dim)  # the configuration BackpropDelta launches: 256x128 tile, eight waves
        else:
            lib.gemm_nt(gt, st, bufs.delta, L.I8, L.I8, k_tile_scale=tsc, k_tile=k_tile, epilogue=L.EPI_ROW_TILE_MAXNORM, tile_scale=bufs.delta_tile_scale)
    ms_dw = event_time_ms(dw, 20)
    avg_ms = (ms_dx + ms_dw) / 2
    roof = {"bound": "mfma", "achieved": gemm_ops / (avg_ms * 1e-3) / 1e12, "peak": PEAK_INT8 / 1e12, "unit": "TFLOP/s",
            "frac": gemm_ops / (avg_ms * 1e-3) / PEAK_INT8,
            # HBM bytes per GEMM launch (mean of the dX and the delta launch) from rocprofv3 FETCH_SIZE / WRITE_SIZE, calibrated against the
            # copy probe (factors 2.0 and 1.0): dX 96.8 + 64.0 MiB, delta 192.3 + 32.0 MiB (two fp32 slices); algorithmic 132.1 and 112.0 MiB
            "traffic": 0.5 * (160.8 + 224.3) * 2 ** 20, "traffic_algorithmic": 0.5 * (132.1 + 112.0) * 2 ** 20,
            "kernel": "GemmNT<int8> (dX launch %.1f us, delta launch %.1f us; 137.44 GOP per launch)" % (ms_dx * 1e3, ms_dw * 1e3)}
    out = {"metric": "fwd+bwd tokens/sec on 1 MI355X; bwd GEMM TFLOPS as % of MFMA peak", "value": len_ / (ms_per_step * 1e-3), "unit": "tokens/s",
           "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": "int8", "data": "synthetic",
           "config": {"workload": "int8 linear-layer backward (dX + delta): X[16384x1024] i8 per-row scales, dY[16384x4096] bf16, W[4096x1024] i8 "
                                  "per-channel scales, k-tile 512", "tokens_per_step": len_, "gemm_gop_per_step": 2 * gemm_ops / 1e9},
           "bwd_gemm_tflops": 2 * gemm_ops / ((ms_dx + ms_dw) * 1e-3) / 1e12, "bwd_gemm_pct_of_peak": 100 * roof["frac"],
           "roofline": roof}
    roof["device_sustained"] = sustained(L.I8)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_linear(len_, src_dim, grad_dim, 4096)
    return out


def _fast_weights(torch, rows, cols, mode_e4m3, gen):
    """random per-matrix quantised weights: N(0,1) * 32 in the 8-bit type (fast = w / (rms/32)), matrix scale 0.02"""
    w = torch.randn((rows, cols), device="cuda", generator=gen) * 32
    if mode_e4m3:
        return w.to(torch.float8_e4m3fn).view(torch.uint8).cpu().numpy(), 0.02
    return torch.clamp(torch.round(w), -128, 127).to(torch.int8).cpu().numpy(), 0.02


def bench_step_fp8(args):
    """BASELINE config[2]: e2048 h16 d12 ffn64 w1024 (24 layers), vocab 50304, 32 sequences x 1024 tokens, e4m3 weights/states/gradients,
    bf16 activations.  One step = forward + loss gradient + backward through all layers with every delta (no optimiser)."""
    import numpy as np
    import torch
    from model_harness import LT_ATT, layer_shapes, schedule
    from oracle_lib import Oracle
    from tscale2_amd import lib as L
    L.load()
    orc = Oracle()
    dim, heads, ffn, depth, vocab, frags, frag_len, wide = 2048, 16, 8192, 12, 50304, 32, 1024, 1024
    if args.small:
        dim, heads, ffn, depth, vocab, frags, frag_len, wide = 512, 4, 2048, 4, 1024, 8, 512, 512
    lt, la, ls, aw = schedule(orc, depth, 0, wide)
    n = frags * frag_len
    m = L.Model(L.E4M3, dim, heads, ffn, lt, la, ls, len(aw), vocab, vocab + 1, n)
    gen = torch.Generator(device="cuda").manual_seed(2)
    params = 0
    for d in range(len(lt)):
        for i, (rows, cols) in enumerate(layer_shapes(int(lt[d]), dim, heads, ffn, 0, 0)):
            fast, sc = _fast_weights(torch, rows, cols, True, gen)
            m.set_matrix(d, i, fast, sc)
            params += rows * cols
    fast, sc = _fast_weights(torch, vocab + 1, dim, True, gen)
    m.set_matrix(L.LAYER_EMBED, 0, fast, sc)
    fast, sc = _fast_weights(torch, vocab, dim, True, gen)
    m.set_matrix(L.LAYER_FINAL, 0, fast, sc)
    params += vocab * dim
    m.set_bias(np.zeros(vocab, np.float32))
    r = np.random.default_rng(3)
    tokens = r.integers(0, vocab, (frags, frag_len))
    tg = np.full((frags, frag_len), -1, np.int32); tg[:, :-1] = tokens[:, 1:]
    t = np.arange(n, dtype=np.int32); frag0 = (t // frag_len) * frag_len
    starts = [np.maximum(frag0, t - int(w)).astype(np.int32) for w in aw]
    finishes = [(t - 1).astype(np.int32) for _ in aw]
    for a in range(len(aw)):
        finishes[a][t == frag0] = -1
    m.set_batch(np.arange(n + 1, dtype=np.int32), (1 + tokens).astype(np.uint32).ravel(), tg.ravel(), starts, finishes, orc.fill_rope_buf(128, n))
    for _ in range(args.warmup):
        m.backprop()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        m.backprop()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    loss = m.loss_sum() / (tg >= 0).sum()
    assert np.isfinite(loss), "loss is not finite"
    # useful work: 6 flop per matmul parameter and token + causal attention (2 fwd + 5 bwd products of S*S/2 x 128 per head)
    att_layers = int((lt == LT_ATT).sum())
    att = 0.0
    for d in range(len(lt)):
        if lt[d] == LT_ATT:
            w = int(aw[la[d]])
            pairs = sum(min(i, w) for i in range(frag_len)) * frags
            att += 7 * 2.0 * pairs * 128 * heads
    flop = 6.0 * params * n + att
    # dominant kernel: the e4m3 GEMM, timed alone on the biggest backward shape of the model (dX of the FFN expand: M=tokens, K=ffn, N=dim)
    a = torch.randint(0, 120, (n, ffn), dtype=torch.uint8, device="cuda"); b = torch.randint(0, 120, (dim, ffn), dtype=torch.uint8, device="cuda")
    c = torch.empty((n, dim), dtype=torch.float32, device="cuda")
    lib = L.load()
    ms_g = event_time_ms(lambda: lib.gemm_nt(a, b, c, L.E4M3, L.F32), 10)
    gops = 2.0 * n * ffn * dim
    roof = {"bound": "mfma", "achieved": gops / (ms_g * 1e-3) / 1e12, "peak": PEAK_FP8 / 1e12, "unit": "TFLOP/s",
            "frac": gops / (ms_g * 1e-3) / PEAK_FP8, "traffic": None,
            "kernel": "GemmNT<e4m3> %dx%dx%d (%.1f us per launch)" % (n, dim, ffn, ms_g * 1e3)}
    out = {"metric": "fwd+bwd tokens/sec on 1 MI355X; bwd GEMM TFLOPS as % of MFMA peak", "value": n / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1,
           "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "fp8_e4m3", "data": "synthetic",
           "config": {"workload": "dense GPT fwd+bwd step, e%dh%dd%dffn%dw%d (%d layers), vocab %d, %d x %d tokens, e4m3 matmuls, bf16 activations"
                                  % (dim, heads, depth, ffn // 128, wide, len(lt), vocab, frags, frag_len),
                      "tokens_per_step": n, "matmul_params": params, "useful_tflop_per_step": flop / 1e12},
           "step_tflops": flop / (ms * 1e-3) / 1e12, "bwd_gemm_pct_of_peak": 100 * roof["frac"], "loss": loss, "roofline": roof}
    roof["device_sustained"] = sustained(L.E4M3)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_step(orc, dim, heads, ffn, lt, la, ls, aw, vocab)
    m.close()
    return out


def cpu_baseline_step(orc, dim, heads, ffn, lt, la, ls, aw, vocab):
    """the oracle's full step (the reference's CPU ComputeBackprop restated) on a bounded sample of the same model: one layer pair
    (attention + FFN) of the real width on 256 tokens, extrapolated per token and per layer"""
    import numpy as np
    from model_harness import Harness
    cores = min(len(os.sched_getaffinity(0)), 16)
    os.environ["OMP_NUM_THREADS"] = str(cores)
    h = Harness(1, dim=dim, heads=heads, ffn_tiles=ffn // 128, depth=1, vocab=256, frag_count=2, frag_len=128, wide_window=128, seed=1)
    t0 = time.perf_counter()
    h.oracle_step()
    dt = time.perf_counter() - t0
    layers_full = len(lt)
    # depth=1 schedule = 1 attention + 1 ffn layer; the full model has layers_full/2 such pairs; the head (vocab) is left out of the sample
    tok_s = h.n / (dt * layers_full / 2)
    return {"value": tok_s, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": "one attention+FFN layer pair of the full width on %d tokens (%.1f s), scaled by %d layer pairs; final layer excluded"
                      % (h.n, dt, layers_full // 2)}


def bench_att_bwd(args):
    """BASELINE config[3]: causal attention backward alone, 16 sequences x 2048, 16 heads x 128, bf16"""
    import torch
    from tscale2_amd import lib as L
    L.load()
    B, S, H = 16, 2048, 16
    n = B * S
    i16 = torch.int16
    gen = torch.Generator(device="cuda").manual_seed(4)
    q, k, v, do = [torch.randn((n, H * 128), device="cuda", generator=gen).bfloat16() for _ in range(4)]
    t = torch.arange(n, device="cuda", dtype=torch.int32)
    start = ((t // S) * S).int().contiguous()
    finish = torch.where(t - 1 >= start, t - 1, torch.full_like(t, -1)).int().contiguous()
    val = torch.empty_like(q); swl = torch.empty((H, n), device="cuda"); ds = torch.zeros((H, n), device="cuda")
    rl = torch.zeros(n // 128, dtype=torch.int32, device="cuda"); rh = torch.zeros_like(rl)
    L.call("ts2_att_build_rev", n, n, start, finish, rl, rh)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    sc = 0.0637
    L.att_forward(n, H, q.view(i16), k.view(i16), v.view(i16), start, finish, sc, 0.0, val.view(i16), swl)
    ds.copy_((val.float() * do.float()).view(n, H, 128).sum(-1).t())

    def step():
        L.att_backward(n, H, q.view(i16), k.view(i16), v.view(i16), do.view(i16), start, finish, rl, rh, sc, 0.0, swl, ds, dq.view(i16), dk.view(i16),
                       dv.view(i16), L.BF16, 3)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ms = event_time_ms(step, args.steps)
    pairs = B * H * (S * (S - 1) / 2)
    flop5 = 5 * 2.0 * pairs * 128
    roof = {"bound": "mfma", "achieved": flop5 / (ms * 1e-3) / 1e12, "peak": PEAK_BF16 / 1e12, "unit": "TFLOP/s", "frac": flop5 / (ms * 1e-3) / PEAK_BF16,
            "traffic": None, "kernel": "AttGradQ + AttGradKV, 5-product causal count (7 products executed)"}
    return {"metric": "fwd+bwd tokens/sec on 1 MI355X; bwd GEMM TFLOPS as % of MFMA peak", "value": n / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16", "data": "synthetic", "config": {"workload": "causal attention backward, 16 x 2048 tokens, 16 heads x 128, bf16"},
            "roofline": roof}


def bench_moe_fp8(args):
    """BASELINE config[4]: one MoE layer forward + backward: 64 experts, top-2, dim 1024, expert width 512, 65536 tokens, e4m3 expert
    weights; the router logits come from a random select matrix on tile-normalised N(0,1) states (mildly imbalanced load).
    One step = ts2_layer_forward + ts2_layer_backward of that layer (routing, gather, grouped expand/gate/contract products, combine,
    routing backward, grouped dX products, grouped deltas, select-matrix backward)."""
    import numpy as np
    import torch
    from tscale2_amd import lib as L
    from oracle_lib import Oracle
    L.load()
    orc = Oracle()
    dim, xp, experts, selected, n, vocab = 1024, 512, 64, 2, 65536, 128
    if args.small:
        n = 8192
    lt = np.array([3], np.int32); la = np.zeros(1, np.int32); ls = np.zeros(1, np.float32)
    # every token carries its own label: the embedding rows are the N(0,1) token states the configuration asks for
    m = L.Model(L.E4M3, dim, 8, 1024, lt, la, ls, 1, vocab, n + 1, n, xp, experts, selected)
    gen = torch.Generator(device="cuda").manual_seed(6)
    shapes = [(xp * experts, dim), (xp * experts, dim), (dim * experts, xp), (experts, dim)]
    for i, (rows, cols) in enumerate(shapes):
        fast, sc = _fast_weights(torch, rows, cols, True, gen)
        # the timed loop re-runs the layer on its own output state: a tiny contract scale keeps that state, and with it the routing,
        # the same in every step (the arithmetic does not depend on the scale)
        m.set_matrix(0, i, fast, 1e-6 if i == 2 else sc)
    fast, sc = _fast_weights(torch, n + 1, dim, True, gen)
    m.set_matrix(L.LAYER_EMBED, 0, fast, sc)
    fast, sc = _fast_weights(torch, vocab, dim, True, gen)
    m.set_matrix(L.LAYER_FINAL, 0, fast, sc)
    m.set_bias(np.zeros(vocab, np.float32))
    r = np.random.default_rng(7)
    tg = r.integers(0, vocab, n).astype(np.int32)
    t = np.arange(n, dtype=np.int32)
    m.set_batch(np.arange(n + 1, dtype=np.int32), (1 + t).astype(np.uint32), tg, [np.maximum(t - 1, 0).astype(np.int32)],
                [(t - 1).astype(np.int32)], orc.fill_rope_buf(128, n))
    m.backprop()                                  # fills state, stateGrad and the gradient scales once

    def step():
        m.layer_forward(0)
        m.layer_backward(0)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ms = event_time_ms(step, args.steps)
    offs = m.read("expertOffset").ravel()
    per_expert = np.diff(offs[:experts + 1])
    routed = n * selected
    flop = 3 * 3 * 2.0 * dim * xp * routed         # three slabs, forward + dX + delta
    # dominant kernel: the grouped e4m3 product; timed alone through the same entry point on a balanced routing of the same size
    lib = L.load()
    rows = routed + 128 * experts
    a = torch.randint(0, 120, (rows, dim), dtype=torch.uint8, device="cuda")
    b = torch.randint(0, 120, (experts * xp, dim), dtype=torch.uint8, device="cuda")
    c = torch.empty((rows, xp), dtype=torch.float32, device="cuda")
    grp = (torch.arange(rows // 128, device="cuda", dtype=torch.int32) * experts // (rows // 128)).int().contiguous()
    ms_g = event_time_ms(lambda: lib.gemm_nt(a, b, c, L.E4M3, L.F32, n=xp, tile_group=grp, b_slab_bytes=xp * dim), 10)
    gops = 2.0 * rows * xp * dim
    roof = {"bound": "mfma", "achieved": gops / (ms_g * 1e-3) / 1e12, "peak": PEAK_FP8 / 1e12, "unit": "TFLOP/s",
            "frac": gops / (ms_g * 1e-3) / PEAK_FP8, "traffic": None,
            "kernel": "GemmNT<e4m3>, expert-grouped rows: %d x %d x %d, %d slabs (%.1f us per launch)" % (rows, xp, dim, experts, ms_g * 1e3)}
    out = {"metric": "fwd+bwd tokens/sec on 1 MI355X; bwd GEMM TFLOPS as % of MFMA peak", "value": n / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1,
           "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "fp8_e4m3", "data": "synthetic",
           "config": {"workload": "MoE layer fwd+bwd: %d experts, top-%d, dim %d, expert width %d, %d tokens, e4m3" % (experts, selected, dim, xp, n),
                      "routed_rows": routed, "useful_tflop_per_step": flop / 1e12,
                      "rows_per_expert_min_mean_max": [int(per_expert.min()), float(per_expert.mean()), int(per_expert.max())]},
           "layer_tflops": flop / (ms * 1e-3) / 1e12, "roofline": roof}
    m.close()
    return out


WORKLOADS = {"linear_i8_bwd": bench_linear_i8, "step_fp8": bench_step_fp8, "att_bwd": bench_att_bwd, "moe_fp8": bench_moe_fp8}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="linear_i8_bwd", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--delta-splits", type=int, default=2, help="linear_i8_bwd: slices of the token axis in the delta product (1 = single pass)")
    ap.add_argument("--small", action="store_true", help="step_fp8 / moe_fp8: a reduced model for quick checks (not a valid benchmark figure)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the path has no multi-GPU leg); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    out = WORKLOADS[args.workload](args)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
