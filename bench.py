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
    bufs = L.MatMulBuffers(L.I8, len_, src_dim, grad_dim, k_tile=k_tile)
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
        lib.gemm_nt(gt, st, bufs.delta, L.I8, L.I8, k_tile_scale=tsc, k_tile=k_tile, epilogue=L.EPI_ROW_TILE_MAXNORM, tile_scale=bufs.delta_tile_scale)
    ms_dw = event_time_ms(dw, 20)
    avg_ms = (ms_dx + ms_dw) / 2
    roof = {"bound": "mfma", "achieved": gemm_ops / (avg_ms * 1e-3) / 1e12, "peak": PEAK_INT8 / 1e12, "unit": "TFLOP/s",
            "frac": gemm_ops / (avg_ms * 1e-3) / PEAK_INT8, "traffic": None,
            "kernel": "GemmNT<int8> (dX launch %.1f us, delta launch %.1f us; 137.44 GOP per launch)" % (ms_dx * 1e3, ms_dw * 1e3)}
    out = {"metric": "fwd+bwd tokens/sec on 1 MI355X; bwd GEMM TFLOPS as % of MFMA peak", "value": len_ / (ms_per_step * 1e-3), "unit": "tokens/s",
           "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": "int8", "data": "synthetic",
           "config": {"workload": "int8 linear-layer backward (dX + delta): X[16384x1024] i8 per-row scales, dY[16384x4096] bf16, W[4096x1024] i8 "
                                  "per-channel scales, k-tile 512", "tokens_per_step": len_, "gemm_gop_per_step": 2 * gemm_ops / 1e9},
           "bwd_gemm_tflops": 2 * gemm_ops / ((ms_dx + ms_dw) * 1e-3) / 1e12, "bwd_gemm_pct_of_peak": 100 * roof["frac"],
           "roofline": roof}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_linear(len_, src_dim, grad_dim, 2048)
    return out


WORKLOADS = {"linear_i8_bwd": bench_linear_i8}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="linear_i8_bwd", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the path has no multi-GPU leg); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    out = WORKLOADS[args.workload](args)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
