#!/usr/bin/env python3
"""Benchmark of the MI355X backward path.  Prints ONE JSON line.

Default workload ("step_fp8") = the dense GPT forward + backward step the metric's tokens/s is quoted on: e2048 h16 d12 ffn64 w1024
(24 layers), vocabulary 50304, 32 sequences x 1024 tokens, e4m3 matmuls with bf16 activations.  One step = forward, loss gradient,
backward through every layer with every packed delta (no optimiser).  The same line carries the second half of the metric, the int8
backward GEMMs of the linear-layer microbenchmark (`bwd_gemm_int8`: X i8 [16384x1024], dY [16384x4096], W i8 [4096x1024]) and the
fused bandwidth kernels' GB/s (`bandwidth_kernels`).  All inputs are resident in HBM before a timed region starts.
Other workloads: "linear_i8_bwd" (that microbenchmark as the step), "att_bwd", "moe_fp8", "bandwidth" (the fused kernels alone) and
"gemm_fp8" (the dominant GEMM alone); the last two end with the copy probe: the commands the HBM-traffic counters are collected on.

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


def settle(fn, ms=40.0):
    """runs fn back to back for about `ms` milliseconds of GPU time, untimed.  After a pause in the launch stream (set-up, allocation,
    a CPU leg) the shader clock needs some 20 ms of load to reach the value it then holds: launches timed before that read 10-25 %
    slow (measured: a 76 us kernel at 114, 93, 84, 80, 79, 77, 76 us over its first blocks of 50 launches).  Every timed region of
    kernels shorter than the warm-up steps of the command line starts behind this."""
    import torch
    torch.cuda.synchronize()
    one = event_time_ms(fn, 1)
    for _ in range(min(4000, int(ms / max(one, 1e-3)))):
        fn()
    torch.cuda.synchronize()


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
    clock = L.probe_shader_clock(lambda: L.probe_mfma_rate(ab_type, 1, 60000), seconds=0.3)
    return {"mfma_only_random_operands_tops": round(L.probe_mfma_rate(ab_type, 1, 100000), 1),
            "mfma_only_random_operands_shader_clock_mhz": round(clock[0]),
            "mfma_only_constant_operands_tops": round(L.probe_mfma_rate(ab_type, 0, 100000), 1),
            "copy_read_plus_write_gbps": round(L.probe_copy_rate(1 << 30), 1)}


def omp_threads(n):
    """thread count of the oracle's OpenMP loops (liboracle.so links libgomp; this is the same runtime instance)"""
    C.CDLL("libgomp.so.1").omp_set_num_threads(int(n))


def host_cores():
    return min(len(os.sched_getaffinity(0)), 16)


def cpu_baseline_linear(len_full, src_dim, grad_dim, sample_rows):
    """The oracle's restatement of the reference CPU path (MulBackwardWithAccum + SumRankOne, cpu_util.cpp:30-67) on a row subsample:
    as written (one thread, a quarter of the sample) and with OpenMP over independent output rows on the host's cores"""
    import numpy as np
    from oracle_lib import Oracle
    orc = Oracle()
    cores = host_cores()
    r = np.random.default_rng(0)
    w = (r.standard_normal((grad_dim, src_dim)) * 0.02).astype(np.float32)
    x = r.standard_normal((sample_rows, src_dim)).astype(np.float32)
    dy = r.standard_normal((sample_rows, grad_dim)).astype(np.float32)

    def run(rows):
        t0 = time.perf_counter()
        orc.mul_backward_accum(np.zeros((rows, src_dim), np.float32), w, dy[:rows])
        orc.sum_rank_one(x[:rows], dy[:rows])
        return time.perf_counter() - t0
    omp_threads(cores)
    dt = run(sample_rows)
    omp_threads(1)
    rows1 = max(sample_rows // 16, 64)
    dt1 = run(rows1)
    omp_threads(cores)
    return {"value": sample_rows / dt, "unit": "rows/s", "cores": cores, "kind": "port",
            "sample": f"{sample_rows} of {len_full} rows (dX + delta, fp32 scalar loops of the reference CPU path, OpenMP over output rows), {dt:.1f} s",
            "single_thread": {"value": rows1 / dt1, "cores": 1, "sample": f"{rows1} rows, {dt1:.1f} s (the reference as written: no threading)"}}


def linear_i8_setup(delta_splits, sort_rows=False):
    """int8 linear-layer workload: tensors and operator buffers of the int8 linear-layer backward"""
    import torch
    from tscale2_amd import lib as L
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
    # the 4096 x 1024 delta has too few tiles for 256 CUs: stored slices of the token axis on 256x128 tiles, packed from their sum
    bufs = L.MatMulBuffers(L.I8, len_, src_dim, grad_dim, k_tile=k_tile, splits=delta_splits, share_row_max=True, sort_rows=sort_rows)
    dx = torch.empty((len_, src_dim), dtype=torch.float32, device="cuda")
    dyv = dy16.view(torch.int16)

    def step():
        # dX = (dY * s_w) W8 : the column scale of W lies on the contraction axis, so it is folded into dY before row quantisation
        bufs.backprop_multi(len_, w8, dyv, L.BF16, w_scale)
        bufs.backprop(len_, None, 1.0, None, dx, L.F32)
        # delta = sum_t (s_x[t] dY[t]) X8[t] : the row scale of X is folded into dY before k-tile quantisation
        bufs.backprop_delta(len_, x8, x_scale, dyv, L.BF16)
    return {"len": len_, "src_dim": src_dim, "grad_dim": grad_dim, "k_tile": k_tile, "splits": delta_splits, "bufs": bufs, "dx": dx, "step": step,
            "x8": x8, "x_scale": x_scale, "w8": w8, "w_scale": w_scale, "dy16": dy16}


def linear_i8_check(c):
    """sanity of both results (not timed): dX and the dequantised packed delta against fp64 products on slices"""
    import torch
    dx, bufs = c["dx"], c["bufs"]
    ref_dx = (c["dy16"][:256].double() * c["w_scale"].double()[None, :]) @ c["w8"].double()
    err = ((dx[:256].double() - ref_dx).abs().max() / ref_dx.abs().max()).item()
    assert err < 3e-2, f"dX deviates from the fp64 product: {err}"
    rows = slice(0, 64)
    ref_dw = (c["dy16"].double()[:, rows] * c["x_scale"].double()[:, None]).t() @ c["x8"].double()
    got = bufs.delta_fp32()[rows].double()
    err = ((got - ref_dw).abs().max() / ref_dw.abs().max()).item()
    assert err < 3e-2, f"the packed delta deviates from the fp64 product: {err}"


def linear_i8_gemm_times(c, iters=20):
    """the two int8 MFMA GEMMs (dX and delta, 137.44 GOP each) timed alone with events on the launch stream"""
    from tscale2_amd import lib as L
    bufs, len_, src_dim, grad_dim, k_tile, splits = c["bufs"], c["len"], c["src_dim"], c["grad_dim"], c["k_tile"], c["splits"]
    dx = lambda: bufs.backprop(len_, None, 1.0, None, c["dx"], L.F32)  # noqa: E731
    settle(dx)
    ms_dx = event_time_ms(dx, iters)
    tsc, gt, st = bufs.t["tileScale"], bufs.t["gradT"], bufs.t["srcT"]
    lib = L.load()

    def dw():
        if splits > 1:
            part = bufs.t["partial"]
            lib.gemm_nt(gt, st, part, L.I8, L.F32, k_tile_scale=tsc, k_tile=k_tile, split_k=splits, split_slab_bytes=grad_dim * src_dim * 4,
                        tile_config=3 | 8, m=grad_dim)  # the configuration BackpropDelta launches: 256x128 tile, eight waves
        else:
            lib.gemm_nt(gt, st, bufs.delta, L.I8, L.I8, k_tile_scale=tsc, k_tile=k_tile, epilogue=L.EPI_ROW_TILE_MAXNORM, tile_scale=bufs.delta_tile_scale)
    settle(dw)
    ms_dw = event_time_ms(dw, iters)
    gemm_ops = 2.0 * len_ * src_dim * grad_dim
    return {"shape": "dY[16384x4096] x W[4096x1024] and dY^T x X[16384x1024], int8 -> int32", "gop_per_launch": gemm_ops / 1e9,
            "dx_us": ms_dx * 1e3, "delta_us": ms_dw * 1e3, "dx_tops": gemm_ops / (ms_dx * 1e-3) / 1e12, "delta_tops": gemm_ops / (ms_dw * 1e-3) / 1e12,
            "tops": 2 * gemm_ops / ((ms_dx + ms_dw) * 1e-3) / 1e12, "frac_of_peak": 2 * gemm_ops / ((ms_dx + ms_dw) * 1e-3) / PEAK_INT8}


def profile_traffic(name):
    """HBM bytes per launch of the dominant kernel as the committed counter summary profiles/<name> states them (a line
    `traffic_bytes_per_launch: N`, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs); None when there is no such summary"""
    path = os.path.join(ROOT, "profiles", name)
    if not os.path.exists(path):
        return None
    for line in open(path):
        if line.startswith("traffic_bytes_per_launch:"):
            return float(line.split(":")[1])
    return None


def bench_linear_i8(args):
    import torch
    from tscale2_amd import lib as L
    L.load()
    c = linear_i8_setup(args.delta_splits, args.sort_rows)
    step, len_ = c["step"], c["len"]
    for _ in range(args.warmup):
        step()
    settle(step)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    linear_i8_check(c)
    g = linear_i8_gemm_times(c)
    gemm_ops = g["gop_per_launch"] * 1e9
    roof = {"bound": "mfma", "achieved": g["tops"], "peak": PEAK_INT8 / 1e12, "unit": "TFLOP/s", "frac": g["frac_of_peak"],
            "traffic": profile_traffic("linear_i8_bwd_hbm_traffic.txt"),
            "kernel": "GemmNT<int8> (dX launch %.1f us, delta launch %.1f us; 137.44 GOP per launch)" % (g["dx_us"], g["delta_us"])}
    out = {"metric": "int8 linear-layer backward rows/sec on 1 MI355X; bwd GEMM TOPS as % of MFMA peak", "value": len_ / (ms_per_step * 1e-3),
           "unit": "rows/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
           "config": {"workload": "int8 linear-layer backward (dX + delta): X[16384x1024] i8 per-row scales, dY[16384x4096] bf16, W[4096x1024] i8 "
                                  "per-channel scales, k-tile 512" + (", rows sorted by scale" if args.sort_rows else ""), "tokens_per_step": len_, "gemm_gop_per_step": 2 * gemm_ops / 1e9},
           "bwd_gemm_tflops": g["tops"], "bwd_gemm_pct_of_peak": 100 * roof["frac"], "bwd_gemm_int8": g, "roofline": roof}
    roof["device_sustained"] = sustained(L.I8)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_linear(len_, c["src_dim"], c["grad_dim"], 4096)
    return out


def _fast_weights(torch, rows, cols, mode_e4m3, gen):
    """random per-matrix quantised weights: N(0,1) * 32 in the 8-bit type (fast = w / (rms/32)), matrix scale 0.02"""
    w = torch.randn((rows, cols), device="cuda", generator=gen) * 32
    if mode_e4m3:
        return w.to(torch.float8_e4m3fn).view(torch.uint8).cpu().numpy(), 0.02
    return torch.clamp(torch.round(w), -128, 127).to(torch.int8).cpu().numpy(), 0.02


def bandwidth_kernels(iters=10, settle_ms=25.0):
    """The fused bandwidth-bound kernels at the shapes of the dense fp8 step (32768 tokens, dim 2048, ffn 8192), of the int8
    linear-layer microbenchmark (16384 x 4096) and of the MoE layer (65536 tokens, top-2 of 64, dim 1024): algorithmic bytes (live
    elements x dtype size of every operand), event time, GB/s and the fraction of the 8 TB/s HBM peak.  Working sets are 0.2-2 GB,
    far beyond the caches."""
    import torch
    from tscale2_amd import lib as L
    dev = "cuda"
    R, D, F = 32768, 2048, 8192
    Q = D
    f32, bf16, u8, i8 = torch.float32, torch.bfloat16, torch.uint8, torch.int8
    res = []
    # (torch's generators are used once before the first launch of this library: under rocprofv3 their first use after it failed with
    # "invalid device function")
    torch.randn(4, device=dev); torch.randint(0, 2, (4,), device=dev); torch.rand(4, device=dev)

    def rnd(rows, cols, dt):
        if dt in (u8,):
            return torch.randint(0, 120, (rows, cols), dtype=u8, device=dev)   # positive finite e4m3 codes
        if dt == i8:
            return torch.randint(-127, 128, (rows, cols), dtype=i8, device=dev)
        return torch.randn((rows, cols), device=dev, dtype=f32).to(dt)

    def add(name, nbytes, fn):
        fn()
        if settle_ms > 0:
            settle(fn, settle_ms)
        ms = event_time_ms(fn, iters)
        res.append({"kernel": name, "mbytes": round(nbytes / 1e6, 1), "us": round(ms * 1e3, 1), "gbps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                    "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / PEAK_HBM, 3)})

    one = torch.ones(4, device=dev)
    # ---- residual state kernels [R][D]
    state = rnd(R, D, f32); norm8 = rnd(R, D, u8); sscale = torch.rand((D // 128, R), device=dev) + 0.5
    add("LayerNormalizeStateVecs f32->e4m3 [32768x2048]", R * D * 5 + R * D // 128 * 4,
        lambda: L.call("ts2_layer_normalize_state_vecs", state, L.F32, R, R, 1 / 24, norm8, L.E4M3, sscale))
    dnorm = rnd(R, D, f32); sgrad = rnd(R, D, f32); sfast = torch.empty((R, D), dtype=u8, device=dev); mx = torch.zeros(4, device=dev)
    add("BackpropLayerNormalize e4m3 [32768x2048]", R * D * 14 + R * D // 128 * 4,
        lambda: L.call("ts2_backprop_layer_normalize", norm8, L.E4M3, sscale, dnorm, None, one, one, sgrad, sfast, L.E4M3, mx, R))
    mx.fill_(1.0)
    add("ScaleGrad f32->e4m3 [32768x2048]", R * D * 5, lambda: L.call("ts2_scale_grad", mx, None, sgrad, sfast, L.E4M3, R, one[1:], one[2:]))
    del state, dnorm, sgrad, sfast, norm8
    # ---- FFN gate kernels [R][F]
    gate = rnd(R, F, bf16); vals = rnd(R, F, bf16); rg = torch.empty((R, F), dtype=u8, device=dev)
    add("MatrixLoLU bf16,bf16->e4m3 [32768x8192]", R * F * 5, lambda: L.call("ts2_matrix_lolu", R, R, gate, vals, 1.0, rg, L.E4M3))
    grad = rnd(R, F, bf16); vts = torch.rand((F // 128, R), device=dev) + 0.5
    gg = torch.empty((R, F), dtype=u8, device=dev); gv = torch.empty_like(gg)
    add("BackpropRowTileNormalizeLoLU bf16,bf16,bf16->e4m3,e4m3 [32768x8192]", R * F * 8 + R * F // 128 * 4,
        lambda: L.call("ts2_backprop_row_tile_normalize_lolu", R, R, gate, vals, 1 / 24, vts, grad, L.BF16, gg, gv, L.E4M3))
    del gate, vals, rg, grad, gg, gv, vts
    # ---- attention epilogue kernels [R][Q]
    gate = rnd(R, Q, bf16); vals = rnd(R, Q, bf16); grad = rnd(R, Q, bf16)
    dgate = torch.empty((R, Q), dtype=u8, device=dev); dval = torch.empty((R, Q), dtype=bf16, device=dev); dsc = torch.empty((Q // 128, R), device=dev)
    add("BackpropLoLUdScale bf16 -> e4m3 + bf16 [32768x2048]", R * Q * 9 + R * Q // 128 * 4,
        lambda: L.call("ts2_backprop_lolu_dscale", R, R, gate, vals, 1.0, grad, L.BF16, dgate, L.E4M3, dval, L.BF16, dsc))
    rope = torch.randn((R, 128), device=dev); qsc = torch.rand((Q // 128, R), device=dev) + 0.5
    add("BackpropRowTileNormalizeRope bf16->e4m3 (norm backward + inverse RoPE) [32768x2048]", R * Q * 5 + R * 128 * 4 + R * Q // 128 * 4,
        lambda: L.call("ts2_backprop_row_tile_normalize_rope", R, R, grad, L.BF16, 1.0, vals, qsc, rope, dgate, L.E4M3))
    raw = rnd(R, Q, f32)
    add("RowTileNormalizeRope f32->bf16 [32768x2048]", R * Q * 6 + R * 128 * 4 + R * Q // 128 * 4,
        lambda: L.call("ts2_row_tile_normalize_rope", R, R, raw, L.F32, 1.0, 1, 1.0, rope, dval, qsc))
    del gate, vals, grad, dgate, dval, raw
    # ---- int8 linear-layer preparation [16384][4096] bf16
    R1, G1, KT = 16384, 4096, 512
    dy = rnd(R1, G1, bf16); d8 = torch.empty((R1, G1), dtype=i8, device=dev); rs = torch.empty(R1, device=dev); ram = torch.empty(R1, device=dev)
    add("NormalizeVecsRowMax bf16->i8 [16384x4096]", R1 * G1 * 3 + R1 * 8,
        lambda: L.call("ts2_normalize_vecs_row_max2", R1, R1, dy, L.BF16, None, d8, rs, ram))
    tmax = torch.zeros(R1 // KT, device=dev); tsc = torch.empty(R1 // KT, device=dev); d8T = torch.empty((G1, R1), dtype=i8, device=dev)
    add("TileAbsMax bf16 [16384x4096]", R1 * G1 * 2, lambda: L.call("ts2_tile_absmax", R1, dy, L.BF16, None, KT, tmax, 1))
    add("TransposeQuant bf16->i8 per k-tile [16384x4096]", R1 * G1 * 3,
        lambda: L.call("ts2_transpose_quant", R1, R1, dy, L.BF16, None, tmax, KT, None, d8T, L.I8, tsc))
    del dy, d8, d8T
    # ---- MoE gradient movement: 65536 tokens, top-2 of 64 experts, dim 1024
    N4, E4, K4, D4 = 65536, 64, 2, 1024
    len_moe = N4 * K4 + 128 * E4
    sel = torch.randn((N4, E4), device=dev)
    tot = N4 * K4
    t = {"ids": torch.zeros(tot, dtype=torch.int32, device=dev), "w": torch.zeros(tot, device=dev), "off": torch.zeros(tot, dtype=torch.int32, device=dev),
         "eo": torch.zeros(E4 + 2, dtype=torch.int32, device=dev), "tile": torch.zeros(len_moe // 128, dtype=torch.int32, device=dev),
         "sid": torch.zeros(len_moe, dtype=torch.int32, device=dev), "sw": torch.zeros(len_moe, device=dev),
         "bc": torch.zeros(((tot + 255) // 256) * E4, dtype=torch.int32, device=dev)}

    class Tables(C.Structure):
        _fields_ = [(n, C.c_void_p) for n in ("ids", "w", "off", "eo", "tile", "sid", "sw", "bc")]
    tb = Tables(*[t[n].data_ptr() for n in ("ids", "w", "off", "eo", "tile", "sid", "sw", "bc")])
    L.call("ts2_moe_route", N4, len_moe, E4, K4, sel, L.F32, C.byref(tb))
    src8 = rnd(N4, D4, u8); grp = torch.empty((len_moe, D4), dtype=u8, device=dev)
    add("MoeGroupSamples 8-bit gather into expert order [131072 of 139264 rows x 1024]", tot * D4 * 2 + len_moe * 4,
        lambda: L.call("ts2_moe_group_samples", len_moe, 1, src8, t["sid"], grp))
    full = rnd(len_moe, D4, bf16); comb = torch.empty((N4, D4), device=dev)
    add("CombineExperts bf16 2-way gather-sum -> f32 [65536x1024]", tot * D4 * 2 + N4 * D4 * 4 + tot * 8,
        lambda: L.call("ts2_combine_experts", N4, K4, full, L.BF16, C.byref(tb), 1.0, None, comb, 0))
    return res


def fp8_backward_gemms(n, dim, ffn, iters=100, warm=20, only_dominant=False):
    """the e4m3 backward GEMM shapes of the dense step, each timed alone with events over `iters` launches after `warm` untimed ones
    and 40 ms more of the same launches (settle()): dX of the FFN contract / expand
    matrices, the FFN delta (packed-delta epilogue) and the attention-width dX"""
    import torch
    from tscale2_amd import lib as L
    lib = L.load()
    out = []

    def run(name, m, nn, k, packed=False, ctype=None):
        if packed:
            # the delta products of the step contract over the rows of both operands as they lie in memory (K-major form)
            a = torch.randint(0, 120, (k, m), dtype=torch.uint8, device="cuda"); b = torch.randint(0, 120, (k, nn), dtype=torch.uint8, device="cuda")
            c = torch.empty((m, nn), dtype=torch.int8, device="cuda"); ts = torch.empty((nn // 128, m), device="cuda")
            fn = lambda: lib.gemm_nt(a, b, c, L.E4M3, L.I8, epilogue=L.EPI_ROW_TILE_MAXNORM, tile_scale=ts, m=m, n=nn, k=k, k_major=True)  # noqa: E731
        else:
            a = torch.randint(0, 120, (m, k), dtype=torch.uint8, device="cuda"); b = torch.randint(0, 120, (nn, k), dtype=torch.uint8, device="cuda")
            c = torch.empty((m, nn), dtype=torch.bfloat16 if ctype == L.BF16 else torch.float32, device="cuda")
            fn = lambda: lib.gemm_nt(a, b, c, L.E4M3, ctype or L.F32)  # noqa: E731
        for _ in range(warm):
            fn()
        settle(fn)
        ms = event_time_ms(fn, iters)
        ops = 2.0 * m * nn * k

        def again():
            for _ in range(iters):
                fn()
        clock = L.probe_shader_clock(again, seconds=ms * iters * 1.3e-3)     # the shader clock while the same launches run once more
        out.append({"product": name, "m": m, "n": nn, "k": k, "us": round(ms * 1e3, 1), "tflops": round(ops / (ms * 1e-3) / 1e12, 1),
                    "frac_of_peak": round(ops / (ms * 1e-3) / PEAK_FP8, 3), "shader_clock_mhz": round(clock[0])})
        return ms, ops
    first = run("dX: dY[tokens x ffn] x W^T (FFN expand / gate), fp32 result", n, dim, ffn)
    if only_dominant:
        return out, first
    run("dX: dY[tokens x dim] x W^T (FFN contract), bf16 result", n, ffn, dim, ctype=L.BF16)
    run("dX: dY[tokens x dim] x W^T (attention Q/K/V/gate/combiner), fp32 result", n, dim, dim)
    run("delta: dY^T[ffn x tokens] x X (FFN expand / gate), both operands token-major, packed i8 result", ffn, dim, n, packed=True)
    run("delta: dY^T[dim x tokens] x X (FFN contract), both operands token-major, packed i8 result", dim, ffn, n, packed=True)
    return out, first


def bench_step_fp8(args):
    """dense fp8 step workload: e2048 h16 d12 ffn64 w1024 (24 layers), vocab 50304, 32 sequences x 1024 tokens, e4m3 weights/states/gradients,
    bf16 activations.  One step = forward + loss gradient + backward through all layers with every delta (no optimiser)."""
    import numpy as np
    import torch
    from tscale2_amd import lib as L
    L.load()
    LT_ATT = 0
    dim, heads, ffn, depth, vocab, frags, frag_len, wide = 2048, 16, 8192, 12, 50304, 32, 1024, 1024
    if args.small:
        dim, heads, ffn, depth, vocab, frags, frag_len, wide = 512, 4, 2048, 4, 1024, 8, 512, 512
    lt, la, ls, aw = L.model_schedule(depth, 0, wide)      # the library's own schedule and RoPE table: no oracle in the timed path
    n = frags * frag_len
    m = L.Model(L.E4M3, dim, heads, ffn, lt, la, ls, len(aw), vocab, vocab + 1, n)
    gen = torch.Generator(device="cuda").manual_seed(2)
    params = 0
    for d in range(len(lt)):
        for i, (rows, cols) in enumerate(L.layer_shapes(int(lt[d]), dim, heads, ffn, 0, 0)):
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
    m.set_batch(np.arange(n + 1, dtype=np.int32), (1 + tokens).astype(np.uint32).ravel(), tg.ravel(), starts, finishes, L.fill_rope_buf(128, n))
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
    # dominant kernel: the e4m3 GEMM, timed alone with events on the launch stream at the model's backward shapes; the roofline line is
    # the biggest of them (dX of the FFN expand / gate matrices: M = tokens, K = ffn, N = dim)
    gemms, (ms_g, gops) = fp8_backward_gemms(n, dim, ffn, only_dominant=args.no_extras)
    roof = {"bound": "mfma", "achieved": gops / (ms_g * 1e-3) / 1e12, "peak": PEAK_FP8 / 1e12, "unit": "TFLOP/s",
            "frac": gops / (ms_g * 1e-3) / PEAK_FP8, "traffic": None if args.small else profile_traffic("gemm_fp8_32768x2048x8192_hbm_traffic.txt"),
            "kernel": "GemmNTRing<e4m3> %dx%dx%d (%.1f us per launch, %.2f GOP)" % (n, dim, ffn, ms_g * 1e3, gops / 1e9)}
    out = {"metric": "fwd+bwd tokens/sec on 1 MI355X; bwd GEMM TFLOPS as % of MFMA peak", "value": n / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1,
           "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "fp8_e4m3", "data": "synthetic",
           "config": {"workload": "dense GPT fwd+bwd step, e%dh%dd%dffn%dw%d (%d layers), vocab %d, %d x %d tokens, e4m3 matmuls, bf16 activations"
                                  % (dim, heads, depth, ffn // 128, wide, len(lt), vocab, frags, frag_len),
                      "tokens_per_step": n, "matmul_params": params, "useful_tflop_per_step": flop / 1e12},
           "step_tflops": flop / (ms * 1e-3) / 1e12, "bwd_gemm_pct_of_peak": 100 * roof["frac"], "loss": loss, "roofline": roof,
           "bwd_gemm_fp8": gemms}
    m.close()
    del m
    torch.cuda.empty_cache()
    if args.no_extras:
        return out
    # the second half of the metric: the int8 backward GEMMs of the linear-layer microbenchmark, in the same run
    c1 = linear_i8_setup(args.delta_splits)
    c1["step"]()
    torch.cuda.synchronize()
    linear_i8_check(c1)
    out["bwd_gemm_int8"] = linear_i8_gemm_times(c1)
    del c1
    torch.cuda.empty_cache()
    out["bandwidth_kernels"] = bandwidth_kernels()
    roof["device_sustained"] = sustained(L.E4M3)
    # config[3] and config[4] beside the step (their own --workload lines carry the CPU legs): a few launches each
    import copy
    sub = copy.copy(args)
    sub.no_cpu, sub.steps, sub.warmup, sub.small = True, 20, 3, False
    a = bench_att_bwd(sub)
    out["att_bwd"] = {"workload": a["config"]["workload"], "ms": a["ms_per_step"], "tokens_per_s": a["value"], "tflops": a["roofline"]["achieved"],
                      "frac_of_bf16_peak": a["roofline"]["frac"], "kernel": a["roofline"]["kernel"], "kernels": a["kernels"]}
    torch.cuda.empty_cache()
    mo = bench_moe_fp8(sub)
    out["moe_layer"] = {"workload": mo["config"]["workload"], "ms": mo["ms_per_step"], "tokens_per_s": mo["value"], "layer_tflops": mo["layer_tflops"],
                        "grouped_product": mo["roofline"]["kernel"], "grouped_product_frac_of_fp8_peak": mo["roofline"]["frac"]}
    torch.cuda.empty_cache()
    if not args.no_cpu:
        from oracle_lib import Oracle            # the CPU leg only
        out["cpu_baseline"] = cpu_baseline_step(Oracle(), dim, heads, ffn, lt, la, ls, aw, vocab)
    return out


def cpu_baseline_step(orc, dim, heads, ffn, lt, la, ls, aw, vocab):
    """the oracle's full step (the reference's CPU ComputeBackprop restated) on a bounded sample of the same model: one layer pair
    (attention + FFN) of the real width on 256 tokens (16 for the single-thread figure), extrapolated per token and per layer"""
    from model_harness import Harness
    cores = host_cores()
    layers_full = len(lt)

    def run(frag_len):
        h = Harness(1, dim=dim, heads=heads, ffn_tiles=ffn // 128, depth=1, vocab=256, frag_count=2, frag_len=frag_len, wide_window=frag_len, seed=1)
        t0 = time.perf_counter()
        h.oracle_step()
        return h.n, time.perf_counter() - t0
    omp_threads(cores)
    n, dt = run(128)
    omp_threads(1)
    n1, dt1 = run(8)
    omp_threads(cores)
    # depth=1 schedule = 1 attention + 1 ffn layer; the full model has layers_full/2 such pairs; the head (vocab) is left out of the sample
    return {"value": n / (dt * layers_full / 2), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": "one attention+FFN layer pair of the full width on %d tokens (%.1f s), scaled by %d layer pairs; final layer excluded"
                      % (n, dt, layers_full // 2),
            "single_thread": {"value": n1 / (dt1 * layers_full / 2), "cores": 1,
                              "sample": "the same pair on %d tokens (%.1f s): the reference as written, no threading" % (n1, dt1)}}


def cpu_baseline_att(heads_full, seqs_full, seq_len):
    """the oracle's attention backward (dScale, GradQ, GradK of layer_att_reference.h restated) on one head of one sequence"""
    import numpy as np
    from oracle_lib import Oracle
    orc = Oracle()
    cores = host_cores()
    r = np.random.default_rng(5)

    def run(s_len):
        q, k, v, do = [r.standard_normal((s_len, 128)).astype(np.float32) for _ in range(4)]
        sp, spans = orc.make_causal_spans(1, s_len, s_len)
        t0 = time.perf_counter()
        orc.attention(1, 128, 128, 0.0, sp, spans, q, k, v, do)
        return time.perf_counter() - t0
    omp_threads(cores)
    dt = run(seq_len)
    omp_threads(1)
    dt1 = run(seq_len // 4)
    omp_threads(cores)
    scale = heads_full * seqs_full
    return {"value": seq_len / (dt * heads_full), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": "forward + backward of 1 head x 1 sequence of %d tokens (%.1f s), scaled by %d heads (x %d sequences = %d head-sequences in the "
                      "workload)" % (seq_len, dt, heads_full, seqs_full, scale),
            "single_thread": {"value": (seq_len // 4) / (dt1 * heads_full * 4), "cores": 1,
                              "sample": "1 head x %d tokens (%.1f s), scaled quadratically to %d tokens per sequence" % (seq_len // 4, dt1, seq_len)}}


def cpu_baseline_moe(dim, xp, experts, selected, tokens):
    """the oracle's MoE layer step (the reference CPU path evaluates every expert densely, layer_moe.cu:458-537) on a token sample"""
    from model_harness import Harness
    cores = host_cores()

    def run(n):
        h = Harness(1, dim=dim, heads=1, ffn_tiles=1, depth=1, vocab=128, frag_count=1, frag_len=n, wide_window=1, experts=experts, selected=selected,
                    xp=xp, seed=1)
        t0 = time.perf_counter()
        h.oracle_step()
        return time.perf_counter() - t0
    omp_threads(cores)
    dt = run(tokens)
    omp_threads(1)
    n1 = max(tokens // 32, 8)
    dt1 = run(n1)
    omp_threads(cores)
    return {"value": tokens / dt, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": "one attention (1 head, window 1) + MoE layer pair, %d experts of width %d evaluated densely, on %d tokens (%.1f s)"
                      % (experts, xp, tokens, dt),
            "single_thread": {"value": n1 / dt1, "cores": 1, "sample": "%d tokens (%.1f s)" % (n1, dt1)}}


def bench_att_bwd(args):
    """attention workload: causal attention backward alone, 16 sequences x 2048, 16 heads x 128, bf16"""
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

    def step(which=3, ds_pair=None):
        L.att_backward(n, H, q.view(i16), k.view(i16), v.view(i16), do.view(i16), start, finish, rl, rh, sc, 0.0, swl, ds, dq.view(i16), dk.view(i16),
                       dv.view(i16), L.BF16, which, ds=ds_pair)
    for _ in range(args.warmup):
        step()
    settle(step)
    ms = event_time_ms(step, args.steps)
    # the two kernels on their own, after the timed region (the device is warm by then)
    ms_dq = event_time_ms(lambda: step(1), args.steps)
    ms_dkdv = event_time_ms(lambda: step(2), args.steps)
    # the optional form with 5 products: dS handed from the dK/dV kernel to a one-product dQ kernel through a scratch array
    pair = L.att_ds_scratch(n, H, start, finish)
    step(3, pair)
    torch.cuda.synchronize()
    ms_five = event_time_ms(lambda: step(3, pair), args.steps)
    ds_mb = pair[1].numel() / 1e6
    del pair
    pairs = B * H * (S * (S - 1) / 2)
    flop5 = 5 * 2.0 * pairs * 128
    roof = {"bound": "mfma", "achieved": flop5 / (ms * 1e-3) / 1e12, "peak": PEAK_BF16 / 1e12, "unit": "TFLOP/s", "frac": flop5 / (ms * 1e-3) / PEAK_BF16,
            "traffic": None, "kernel": "AttGradQ + AttGradKV, 5-product causal count (7 products executed: S and dP once per kernel)"}
    out = {"metric": "attention backward tokens/sec on 1 MI355X; TFLOPS as % of MFMA peak", "value": n / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1,
           "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "bf16", "data": "synthetic", "config": {"workload": "causal attention backward, 16 x 2048 tokens, 16 heads x 128, bf16"},
           "roofline": roof, "kernels": {"dq_ms": ms_dq, "dkdv_ms": ms_dkdv, "dq_products": 3, "dkdv_products": 4},
           "five_products": {"ms": ms_five, "scratch_mbytes": ds_mb,
                             "note": "ts2_att_grad_args.dsScratch: dS leaves the dK/dV kernel as bf16 blocks, dQ is one product over them"}}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_att(H, B, S)
    return out


def bench_moe_fp8(args):
    """MoE workload: one MoE layer forward + backward: 64 experts, top-2, dim 1024, expert width 512, 65536 tokens, e4m3 expert
    weights; the router logits come from a random select matrix on tile-normalised N(0,1) states (mildly imbalanced load).
    One step = ts2_layer_forward + ts2_layer_backward of that layer (routing, gather, grouped expand/gate/contract products, combine,
    routing backward, grouped dX products, grouped deltas, select-matrix backward)."""
    import numpy as np
    import torch
    from tscale2_amd import lib as L
    L.load()
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
                [(t - 1).astype(np.int32)], L.fill_rope_buf(128, n))
    m.backprop()                                  # fills state, stateGrad and the gradient scales once

    def step():
        m.layer_forward(0)
        m.layer_backward(0)
    for _ in range(args.warmup):
        step()
    settle(step)
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
    c = torch.empty((rows, xp), dtype=torch.bfloat16, device="cuda")   # 16-bit results, as every grouped product of the layer stores them
    grp = (torch.arange(rows // 128, device="cuda", dtype=torch.int32) * experts // (rows // 128)).int().contiguous()
    grouped = lambda: lib.gemm_nt(a, b, c, L.E4M3, L.BF16, n=xp, tile_group=grp, b_slab_bytes=xp * dim)
    settle(grouped)
    ms_g = event_time_ms(grouped, 300)
    gops = 2.0 * rows * xp * dim
    roof = {"bound": "mfma", "achieved": gops / (ms_g * 1e-3) / 1e12, "peak": PEAK_FP8 / 1e12, "unit": "TFLOP/s",
            "frac": gops / (ms_g * 1e-3) / PEAK_FP8, "traffic": None,
            "kernel": "GemmNT<e4m3>, expert-grouped rows, bf16 result: %d x %d x %d, %d slabs (%.1f us per launch)" % (rows, xp, dim, experts, ms_g * 1e3)}
    out = {"metric": "fwd+bwd tokens/sec on 1 MI355X; bwd GEMM TFLOPS as % of MFMA peak", "value": n / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1,
           "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "fp8_e4m3", "data": "synthetic",
           "config": {"workload": "MoE layer fwd+bwd: %d experts, top-%d, dim %d, expert width %d, %d tokens, e4m3" % (experts, selected, dim, xp, n),
                      "routed_rows": routed, "useful_tflop_per_step": flop / 1e12,
                      "rows_per_expert_min_mean_max": [int(per_expert.min()), float(per_expert.mean()), int(per_expert.max())]},
           "layer_tflops": flop / (ms * 1e-3) / 1e12, "roofline": roof}
    m.close()
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_moe(dim, xp, experts, selected, 256)
    return out


def bench_gemm_fp8(args):
    """one e4m3 product alone - by default the dominant kernel of the dense fp8 step (32768 x 2048 x 8192, fp32 result) - followed by the
    copy probe of 1 GiB: the command the hardware counters (rocprofv3 --pmc) are collected on; the probe calibrates FETCH_SIZE / WRITE_SIZE.
    --shape m,n,k, --result f32|bf16|norm and --tile-config (ts2_gemm_args.tileConfig: 32768 = never the persistent kernel, 4096 = always)
    select other products of the step; the shader clock is sampled while the launches run."""
    import torch
    from tscale2_amd import lib as L
    lib = L.load()
    n, dim, ffn = [int(x) for x in args.shape.split(",")] if args.shape else (32768, 2048, 8192)
    a = torch.randint(0, 120, (n, ffn), dtype=torch.uint8, device="cuda"); b = torch.randint(0, 120, (dim, ffn), dtype=torch.uint8, device="cuda")
    kw = {"tile_config": args.tile_config}
    if args.result == "f32":
        c = torch.empty((n, dim), dtype=torch.float32, device="cuda")
        ct = L.F32
    else:
        c = torch.empty((n, dim), dtype=torch.int16, device="cuda")
        ct = L.BF16
        if args.result == "norm":
            kw.update(epilogue=L.EPI_ROW_TILE_NORM, normalize=True, vec_scale=1 / 24.0, tile_scale=torch.empty((dim // 128, n), device="cuda"))
    fn = lambda: lib.gemm_nt(a, b, c, L.E4M3, ct, **kw)  # noqa: E731
    for _ in range(args.warmup):
        fn()
    settle(fn)
    ms = event_time_ms(fn, args.steps)
    gops = 2.0 * n * dim * ffn
    reps = max(20, int(40.0 / ms))

    def many():
        for _ in range(reps):
            fn()
    clock = L.probe_shader_clock(many, seconds=reps * ms * 1.3e-3)
    copy = L.probe_copy_rate(1 << 30)
    default = not args.shape and args.result == "f32"
    roof = {"bound": "mfma", "achieved": gops / (ms * 1e-3) / 1e12, "peak": PEAK_FP8 / 1e12, "unit": "TFLOP/s", "frac": gops / (ms * 1e-3) / PEAK_FP8,
            "traffic": profile_traffic("gemm_fp8_32768x2048x8192_hbm_traffic.txt") if default else None,
            "traffic_algorithmic": n * ffn + dim * ffn + n * dim * (4 if ct == L.F32 else 2),
            "kernel": "e4m3 GEMM %dx%dx%d, %s result, tileConfig %d" % (n, dim, ffn, args.result, args.tile_config),
            "shader_clock_mhz_median_min_max": clock}
    return {"metric": "e4m3 GEMM launches/sec on 1 MI355X; TFLOPS as % of MFMA peak", "value": 1e3 / ms, "unit": "launches/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "fp8_e4m3", "data": "synthetic", "config": {"workload": "e4m3 GEMM %d x %d x %d, %s result" % (n, dim, ffn, args.result)},
            "copy_probe_gbps": copy, "roofline": roof}


def bench_bandwidth(args):
    """the fused bandwidth-bound kernels alone, followed by the copy probe of 1 GiB: the command their HBM counters (rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE) are collected on; the probe calibrates the counters.  `value` is the byte-weighted rate of the set.
    With --steps below 5 the kernels are launched --steps times each after one warm-up launch and no settling loop (counter runs)."""
    from tscale2_amd import lib as L
    L.load()
    few = args.steps < 5
    res = bandwidth_kernels(iters=max(1, args.steps), settle_ms=0.0 if few else 25.0)
    copy = L.probe_copy_rate(1 << 30)
    nbytes = sum(r["mbytes"] for r in res) * 1e6
    secs = sum(r["us"] for r in res) * 1e-6
    worst = min(res, key=lambda r: r["frac_of_hbm_peak"])
    roof = {"bound": "hbm", "achieved": nbytes / secs / 1e9, "peak": PEAK_HBM / 1e9, "unit": "GB/s", "frac": nbytes / secs / PEAK_HBM, "traffic": None,
            "kernel": "all %d kernels, byte-weighted; lowest: %s (%.3f)" % (len(res), worst["kernel"], worst["frac_of_hbm_peak"])}
    return {"metric": "fused gradient kernels, algorithmic GB/s on 1 MI355X as % of HBM peak", "value": nbytes / secs / 1e9, "unit": "GB/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": secs * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "mixed (fp32 / bf16 / e4m3 / int8 streams)", "data": "synthetic",
            "config": {"workload": "the 13 fused bandwidth-bound kernels at the shapes of configs 1, 2 and 4, one launch series each"},
            "copy_probe_gbps": copy, "bandwidth_kernels": res, "roofline": roof}


WORKLOADS = {"linear_i8_bwd": bench_linear_i8, "step_fp8": bench_step_fp8, "att_bwd": bench_att_bwd, "moe_fp8": bench_moe_fp8,
             "gemm_fp8": bench_gemm_fp8, "bandwidth": bench_bandwidth}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="step_fp8", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--delta-splits", type=int, default=2, help="linear_i8_bwd: slices of the token axis in the delta product (1 = single pass)")
    ap.add_argument("--sort-rows", action="store_true", help="linear_i8_bwd: sort the gradient rows by scale before the delta product (the reference's order)")
    ap.add_argument("--no-extras", action="store_true", help="step_fp8: only the step and its dominant GEMM (no int8 GEMMs, bandwidth kernels, device "
                                                              "probes or CPU leg): the command a kernel trace of the step is taken on")
    ap.add_argument("--shape", default="", help="gemm_fp8: m,n,k of the product (default 32768,2048,8192)")
    ap.add_argument("--result", default="f32", choices=["f32", "bf16", "norm"], help="gemm_fp8: fp32 store, bf16 store, or row-tile normalised bf16")
    ap.add_argument("--tile-config", type=int, default=0, help="gemm_fp8: ts2_gemm_args.tileConfig")
    ap.add_argument("--small", action="store_true", help="step_fp8 / moe_fp8: a reduced model for quick checks (not a valid benchmark figure)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (no collective, sharding or rank code is part of it): run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    out = WORKLOADS[args.workload](args)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
