#!/usr/bin/env python3
"""Benchmark of the MXFP6 GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" = one pass of the operator over one batch of synthetic inputs that already sit in HBM:
C[8192,8192] (bf16) = A[8192,8192] . B[8192,8192]^T with MXFP6 e2m3 operands (BASELINE.json
configs[1]: N(0,1) sources, per-32 E8M0 scales).  Sources are drawn on the CPU (numpy default_rng with
the seeds of SEEDS, so the bytes do not depend on the torch build), uploaded and quantised with the
library's own quantise+pack kernel (bit-exact against the CPU oracle by the tests); the timed loop
cycles through several independent input sets, the counterpart of the reference protocol's fresh
inputs per iteration (kernels/gemm/bf16fp32/utils.py:36-54: warm-up launches, then timed launches
bracketed by device events, TFLOPS = 2*M*N*K / t).

Prints ONE JSON line.  `value` is TFLOP/s of the whole job on row-major inputs (wall clock between two
device synchronisations / steps; a step includes the library's re-layout pre-pass of both operands);
`value_prepared_weights` is the same step with B converted to the tile-major weight format once,
outside the timed region (the pre-pass then copies A only).  `roofline` prices the tiled GEMM kernel
alone against the dense MXFP6 MFMA peak using the mean per-launch duration measured with device events
on the launch stream.  `configs` holds every BASELINE.json configuration with its own operand
distributions and formats: time, TFLOPS or GB/s, fraction of the roof, accuracy on sampled rows against
the CPU oracle, and a CPU baseline in two forms (the OpenMP C port of dequantise-and-matmul, and
dequantise + torch.matmul in fp32 timed separately).  `decode` details the M=16 skinny kernel
(configs[3]) and batched decode against the HBM peak, `quantize` the quantise+pack kernel.
`cpu_baseline` is the configs[1] leg; it is a reported baseline, not a target.

The ceilings and ablations (`roofline.sustained`, `decode.roofline.stream_probe`) come from the
measurement build of the library (libmxfp6_probes.so, include/mxfp6_probes.h); every other figure is the
operator's own library.
"""
from __future__ import annotations

import argparse
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MFMA_PEAK_TFLOPS = 10066.0  # MI355X dense MXFP6: 256 CU x 4 SIMD x 4096 FLOP/clk x 2.4 GHz
HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
PUBLISHED_FP6_8192 = 2861.52  # reference's published FP6 GEMM at 8192^3 on MI355X (analysis/fp6_gemm/mi355x_fp6_gemm.json:5)
# the other square sizes of the same published table (analysis/fp6_gemm/mi355x_fp6_gemm.json:2-6), TFLOPS
PUBLISHED_FP6_SQUARES = {1024: 74.9089, 2048: 470.161, 4096: 1865.47, 16384: 3122.13}
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "traffic.json")
# the sources whose text decides what the two profiled kernels move; profiles/traffic.json records their hash
TRAFFIC_SOURCES = {"gemm_tiled_kernel": ("gemm_tiled.hip", "common.hpp", "loader.hpp"), "gemm_skinny_kernel": ("gemm_skinny.hip", "common.hpp", "loader.hpp"),
                   "gemm_ring_kernel_m16": ("gemm_ring.hip", "common.hpp", "loader.hpp"), "gemm_ring_kernel_m64": ("gemm_ring.hip", "common.hpp", "loader.hpp")}
# kernel behind a code of tk_kernel.kernel_choice, for the decode shapes
DECODE_KERNELS = {3: "gemm_skinny_kernel", 28: "gemm_ring_kernel", 22: "gemm_block_kernel", 26: "gemm_block_kernel", 27: "gemm_block_kernel", 2: "gemm_tiled_kernel", 25: "gemm_tiled_kernel", 1: "gemm_generic_kernel"}

# BASELINE.json configs: shape, formats, source distributions (A, B), seed
CONFIGS = {
    "cfg0": dict(M=256, N=256, K=256, fa=2, fb=2, kind_a="normal", kind_b="normal", seed=0, bound="mfma"),
    "cfg1": dict(M=8192, N=8192, K=8192, fa=2, fb=2, kind_a="normal", kind_b="normal", seed=1, bound="mfma"),
    "cfg2": dict(M=4096, N=28672, K=8192, fa=2, fb=2, kind_a="normal", kind_b="weights_outliers", seed=2, bound="mfma"),
    "cfg3": dict(M=16, N=8192, K=28672, fa=2, fb=2, kind_a="normal", kind_b="weights", seed=3, bound="hbm"),
    "cfg4": dict(M=8192, N=8192, K=16384, fa=3, fb=2, kind_a="laplace", kind_b="weights", seed=4, bound="mfma"),
}
FMT_NAME = {2: "e2m3", 3: "e3m2"}


def algorithmic_bytes(M, N, K):
    return 0.75 * K * (M + N) + (K // 32) * (M + N) + 2 * M * N


def cpu_source(kind, shape, seed):
    """fp32 sources of BASELINE.json's configurations, drawn on the CPU."""
    import numpy as np

    rng = np.random.default_rng(seed)
    if kind == "normal":
        return rng.standard_normal(shape, dtype=np.float32)
    if kind == "weights":
        return rng.standard_normal(shape, dtype=np.float32) * np.float32(0.02)
    if kind == "weights_outliers":  # N(0, 0.02), 1 % of the entries multiplied by 8
        w = rng.standard_normal(shape, dtype=np.float32) * np.float32(0.02)
        w[rng.random(shape, dtype=np.float32) < 0.01] *= np.float32(8.0)
        return w
    if kind == "laplace":
        return rng.laplace(0.0, 1.0, shape).astype(np.float32)
    raise ValueError(kind)


def quantised(hk, torch, kind, rows, K, fmt, seed, copies=1):
    """`copies` quantised operands from one CPU-drawn source: the source itself, then the source with its rows rotated
    (other bytes at every address, the same distribution), so that a timed loop cycles through distinct memory."""
    x = torch.from_numpy(cpu_source(kind, (rows, K), seed)).cuda()
    out = []
    for c in range(copies):
        out.append(hk.quantize(x if c == 0 else torch.roll(x, shifts=c * 37 + 1, dims=0), fmt))
    del x
    return out


def make_inputs(hk, torch, cfg, sets):
    a = quantised(hk, torch, cfg["kind_a"], cfg["M"], cfg["K"], cfg["fa"], 1000 * cfg["seed"] + 1, sets)
    b = quantised(hk, torch, cfg["kind_b"], cfg["N"], cfg["K"], cfg["fb"], 1000 * cfg["seed"] + 2, sets)
    torch.cuda.synchronize()
    return [(a[i][0], b[i][0], a[i][1], b[i][1]) for i in range(sets)]


def tiled(hk, ops, K, which="ab"):
    ap, bp, asc, bsc = ops
    if "a" in which:
        ap, asc = hk.tile_operand(ap), hk.tile_scales(asc, K)
    if "b" in which:
        bp, bsc = hk.tile_operand(bp), hk.tile_scales(bsc, K)
    return ap, bp, asc, bsc


PREWARM_MS = 40.0  # see timed_loop


def timed_loop(hk, torch, inputs, C, steps, warmup, layout_a=0, layout_b=0, prewarm_ms=0.0, fa=2, fb=2, call=None):
    """W untimed + K timed launches.  Returns (wall seconds for the K steps between two device
    synchronisations, mean per-launch milliseconds from one pair of device events recorded on the
    launch stream around the K back-to-back launches).
    prewarm_ms > 0: before the W warm-up steps the same launches run untimed for that long.  The chip's power
    management takes tens of milliseconds to settle under this load (launch durations by rocprofv3 kernel-trace at
    8192^3: ~290 us for the first ~8 launches after idle, 340-370 us from the 10th to the 25th, back to ~295 us from about
    the 45th on), so a short W + K would time the transient instead of the kernel.
    call: what launches one step (default: the operator, hk.dispatch_micro)."""
    n = len(inputs)
    if call is None:
        def call(ops):
            hk.dispatch_micro(ops[0], ops[1], ops[2], ops[3], C, fa, fb, layout_a=layout_a, layout_b=layout_b)
    if prewarm_ms > 0:
        t_end = time.perf_counter() + prewarm_ms * 1e-3
        i = 0
        while time.perf_counter() < t_end:
            for _ in range(8):
                call(inputs[i % n])
                i += 1
            torch.cuda.synchronize()
    for i in range(warmup):
        call(inputs[i % n])
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        call(inputs[i % n])
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, e0.elapsed_time(e1) / steps


def per_launch_ref_protocol(hk, torch, M, N, K, iters, seed):
    """The reference harness's protocol (kernels/gemm/bf16fp32/utils.py:36-50): fresh random inputs for every
    iteration (drawn on the device here: thousands of CPU draws of 8192 x 8192 would take minutes), a device
    synchronisation, and one pair of device events around each single launch.  Returns per-launch milliseconds (median,
    mean) of (a) the operator on row-major inputs, pre-pass included, and (b) the tiled kernel alone on the tile-major
    operands the quantiser emits directly."""
    import statistics

    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    C = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    xa = torch.empty(M, K, device="cuda", dtype=torch.float32)
    xb = torch.empty(N, K, device="cuda", dtype=torch.float32)
    t_op, t_k = [], []
    for it in range(iters + 3):
        xa.normal_(generator=g)
        xb.normal_(generator=g)
        ap, asc = hk.quantize(xa, 2)
        bp, bsc = hk.quantize(xb, 2)
        at, ast = hk.quantize(xa, 2, layout=hk.LAYOUT_TILE)
        bt, bst = hk.quantize(xb, 2, layout=hk.LAYOUT_TILE)
        for lay, ops, acc in ((0, (ap, bp, asc, bsc), t_op), (1, (at, bt, ast, bst), t_k)):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            hk.dispatch_micro(*ops, C, layout_a=lay, layout_b=lay)
            e1.record()
            torch.cuda.synchronize()
            if it >= 3:  # the first iterations take the one-time costs (workspace, code load)
                acc.append(e0.elapsed_time(e1))
    return {"operator_row_major_ms_median": statistics.median(t_op), "operator_row_major_ms_mean": statistics.fmean(t_op),
            "kernel_tile_major_ms_median": statistics.median(t_k), "kernel_tile_major_ms_mean": statistics.fmean(t_k), "iters": iters}


def _clock_ghz(stats):
    clk, rt = (int(stats[2]) - int(stats[0])) & 0xFFFFFFFF, (int(stats[3]) - int(stats[1])) & 0xFFFFFFFF
    return (clk / (rt * 10.0) if rt else 0.0), clk  # real-time counter: 100 MHz


def probes(hk, torch, P, inputs, kinputs, C, M, N, K):
    """What the silicon sustains, measured with the measurement build's probe kernels on this run's own operand bytes,
    next to (not instead of) the nominal peaks: the scaled-MFMA issue rate and shader clock with every other unit idle,
    the tiled kernel's own shader clock, the same kernel on all-zero operands (the clock stays up: the gap to the
    real-data run is power management, not the schedule), and builds of the kernel without one of its parts."""
    stream = torch.cuda.current_stream().cuda_stream
    ap, bp, asc, bsc = inputs[0]
    stats = torch.zeros(4, dtype=torch.int32, device="cuda")
    sink = torch.zeros(1, dtype=torch.float32, device="cuda")
    out = {}
    iters = 8192
    for name, a, b, sa, sb in (("real_operands", ap, bp, asc, bsc),
                               ("zero_operands", torch.zeros_like(ap), torch.zeros_like(bp), torch.full_like(asc, 127), torch.full_like(bsc, 127))):
        def launch():
            return P.mxfp6_probe_mfma(a.data_ptr(), b.data_ptr(), sa.data_ptr(), sb.data_ptr(), M, N, K, 2, 2, iters, sink.data_ptr(), stats.data_ptr(), stream)
        # the same settling time as the GEMM loops get: under this load the clock takes tens of milliseconds to find its level
        t_end = time.perf_counter() + PREWARM_MS * 1e-3
        while time.perf_counter() < t_end:
            waves = launch()
            torch.cuda.synchronize()
        assert waves > 0, waves
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(5):
            launch()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / 5
        ghz, clk = _clock_ghz(stats.cpu().numpy())
        out["mfma_only_" + name] = {"tflops": waves * 4.0 * iters * 131072 / (ms * 1e-3) / 1e12, "launch_ms": ms, "shader_clock_ghz": ghz}

    # the tiled kernel through the measurement build (the same kernel source; the operator's library has no overrides)
    def call(ops):
        rc = P.mxfp6_gemm_ex(ops[0].data_ptr(), ops[1].data_ptr(), ops[2].data_ptr(), ops[3].data_ptr(), C.data_ptr(), M, N, K, 2, 2, 1, 1, 0, stream)
        assert rc == 0, rc
    assert P.mxfp6_probe_tiled_clock(stats.data_ptr()) == 0
    prev = P.mxfp6_set_relayout(0)
    try:
        for name, ops in (("real_operands", kinputs[0]),
                          ("zero_operands", (torch.zeros_like(kinputs[0][0]), torch.zeros_like(kinputs[0][1]), torch.full_like(kinputs[0][2], 127), torch.full_like(kinputs[0][3], 127)))):
            _, ms = timed_loop(hk, torch, [ops], C, 20, 10, prewarm_ms=PREWARM_MS, call=call)
            ghz, clk = _clock_ghz(stats.cpu().numpy())
            out["tiled_kernel_" + name] = {"launch_ms_mean": ms, "tflops": 2.0 * M * N * K / (ms * 1e-3) / 1e12, "shader_clock_ghz": ghz,
                                           "clocks_per_k_tile": clk / ((M // 256) * (N // 256) / 256.0 * (K // 128))}
        # what each part of the kernel costs: builds of the same kernel without its LDS reads (1), its loads (2), its MFMAs (4)
        abl = {}
        names = {0: "full", 1: "no_lds_reads", 2: "no_loads", 3: "mfma_only", 4: "no_mfma", 6: "lds_reads_only", 8: "full_plus_idle_clocks"}
        for mask in (0, 1, 2, 3, 4, 6, 8, 0):
            assert P.mxfp6_probe_tiled_ablation(mask) == 0
            _, ms = timed_loop(hk, torch, [kinputs[0]], C, 20, 10, prewarm_ms=PREWARM_MS if mask in (0, 3, 8) else 0.0, call=call)
            ghz, clk = _clock_ghz(stats.cpu().numpy())
            abl[names[mask]] = {"launch_ms_mean": ms, "shader_clock_ghz": ghz, "kclocks": clk / 1e3}
        # the same two builds on all-zero operands, where nothing is power-limited: there the idle clocks cost their time
        zops = (torch.zeros_like(kinputs[0][0]), torch.zeros_like(kinputs[0][1]), torch.full_like(kinputs[0][2], 127), torch.full_like(kinputs[0][3], 127))
        for mask in (8, 0):
            assert P.mxfp6_probe_tiled_ablation(mask) == 0
            _, ms = timed_loop(hk, torch, [zops], C, 20, 10, prewarm_ms=PREWARM_MS, call=call)
            ghz, clk = _clock_ghz(stats.cpu().numpy())
            abl[names[mask] + "_zero_operands"] = {"launch_ms_mean": ms, "shader_clock_ghz": ghz, "kclocks": clk / 1e3}
        del zops
        out["tiled_kernel_ablations"] = abl
        # the builds with MFMAs run at a power-managed clock: what adding a part costs there, in time
        t = {k: v["launch_ms_mean"] * 1e3 for k, v in abl.items()}
        out["power_limited_time_split_us"] = {
            "mfma_only": t["mfma_only"], "lds_reads_added": t["no_loads"] - t["mfma_only"], "loads_added": t["no_lds_reads"] - t["mfma_only"],
            "rest": t["full"] - t["no_loads"] - t["no_lds_reads"] + t["mfma_only"], "full": t["full"],
            "what": "launch time (us) of the MFMA-only build, what the LDS reads and what the direct loads add to it when added alone, and what is left of the full kernel's time",
        }
        out["mfma_only_build_tflops"] = 2.0 * M * N * K / (t["mfma_only"] * 1e-6) / 1e12
    finally:
        P.mxfp6_set_relayout(prev)
        P.mxfp6_probe_tiled_clock(None)
        P.mxfp6_probe_tiled_ablation(0)
    return out


def stream_probe(torch, P):
    """A kernel that only reads: 2 GiB once through direct-to-LDS loads, nothing else (no arithmetic, no stores)."""
    stream = torch.cuda.current_stream().cuda_stream
    buf = torch.empty(1 << 31, dtype=torch.uint8, device="cuda")
    buf.view(torch.int32).random_()
    stats = torch.zeros(4, dtype=torch.int32, device="cuda")
    best, tried = None, {}
    for wgs, waves in ((256, 8), (512, 8), (1024, 8), (512, 4), (1024, 4), (2048, 4)):
        for _ in range(2):
            rc = P.mxfp6_probe_stream(buf.data_ptr(), buf.numel(), wgs, waves, stats.data_ptr(), stream)
            assert rc == 0, rc
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(5):
            P.mxfp6_probe_stream(buf.data_ptr(), buf.numel(), wgs, waves, stats.data_ptr(), stream)
        e1.record()
        torch.cuda.synchronize()
        gbs = buf.numel() / (e0.elapsed_time(e1) / 5 * 1e-3) / 1e9
        tried[f"{wgs}x{waves}"] = gbs
        if best is None or gbs > best[0]:
            best = (gbs, wgs, waves)
    del buf
    return {"stream_ceiling_gbs": best[0], "workgroups": best[1], "waves_per_workgroup": best[2], "bytes": 1 << 31, "tried_gbs": tried,
            "what": "read-only kernel, 2 GiB once (8x the 256 MB last-level cache), direct-to-LDS loads, 16 KB in flight per wave; best of the launch shapes tried"}


def cpu_legs(cfg, ops, rows, k_slice, gpu_f32):
    """The CPU baseline on this run's own bytes, in two forms: the OpenMP C port of
    dequantise-and-matmul (oracle/mxfp6_oracle.c) and dequantise (the C oracle's) + torch.matmul in fp32, each part timed.
    rows: the first `rows` rows of A; k_slice: the first K / k_slice columns of K (1 = all of K).  gpu_f32: the library's
    fp32 result for the same rows over the same K range, compared with the C port's with the parity metric."""
    import numpy as np
    import torch

    from oracle import c_oracle as co
    from oracle import mxfp6_oracle as o

    ap, bp, asc, bsc = ops
    K = cfg["K"] // k_slice
    ap_h, asc_h = ap[:rows, : K // 4 * 3].contiguous().cpu().numpy(), asc[:rows, : K // 32].contiguous().cpu().numpy()
    bp_h, bsc_h = bp[:, : K // 4 * 3].contiguous().cpu().numpy(), bsc[:, : K // 32].contiguous().cpu().numpy()
    N = bp_h.shape[0]
    flops = 2.0 * rows * N * K
    t0 = time.perf_counter()
    ref = co.gemm_f32(ap_h, bp_h, asc_h, bsc_h, cfg["fa"], cfg["fb"])
    t_port = time.perf_counter() - t0
    t0 = time.perf_counter()
    a32 = torch.from_numpy(co.dequantise(ap_h, asc_h, cfg["fa"]))
    b32 = torch.from_numpy(co.dequantise(bp_h, bsc_h, cfg["fb"]))
    t_dq = time.perf_counter() - t0
    t0 = time.perf_counter()
    c_t = torch.matmul(a32, b32.t())
    t_mm = time.perf_counter() - t0
    sample = f"first {rows} of {cfg['M']} rows of A against all {N} rows of B, " + ("all of K" if k_slice == 1 else f"the first 1/{k_slice} of K ({K} of {cfg['K']}), a slice and labelled so")
    out = {
        "port": {"value": flops / t_port / 1e12, "unit": "TFLOPS", "seconds": t_port, "cores": co.num_threads(), "kind": "port", "what": "OpenMP C restatement of dequantise-and-matmul"},
        "torch_matmul": {"value": flops / (t_dq + t_mm) / 1e12, "unit": "TFLOPS", "dequantise_seconds": t_dq, "matmul_seconds": t_mm, "cores": torch.get_num_threads(),
                         "kind": "port", "what": "dequantise to fp32 (C oracle) + torch.matmul on the host cores, timed separately",
                         "max_rel_err_vs_port": o.rel_err(c_t.numpy(), ref)},
        "sample": sample, "k_slice": k_slice,
    }
    if gpu_f32 is not None:
        out["max_rel_err_gpu_vs_cpu"] = o.rel_err(gpu_f32, ref)
        out["max_rel_err_bar"] = 2e-3
    return out


def run_config(hk, torch, name, steps, warmup, cpu, sets=2):
    """One BASELINE.json configuration with its own distributions and formats: the operator on row-major inputs and on
    tile-major operands (back-to-back launches, device events), accuracy on rows of the fp32 result against the CPU
    oracle, CPU baseline (all of cfg0 / cfg3, a labelled 1/8-K slice of cfg2 / cfg4)."""
    cfg = CONFIGS[name]
    M, N, K, fa, fb = cfg["M"], cfg["N"], cfg["K"], cfg["fa"], cfg["fb"]
    ins = make_inputs(hk, torch, cfg, sets)
    C = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    pre = PREWARM_MS if cfg["bound"] == "mfma" and M >= 4096 else 0.0
    _, row_ms = timed_loop(hk, torch, ins, C, steps, warmup, 0, 0, prewarm_ms=pre, fa=fa, fb=fb)
    tile_ms = None
    if M % 32 == 0 and N % 32 == 0 and K % 128 == 0:
        tins = [tiled(hk, ops, K) for ops in ins]
        _, tile_ms = timed_loop(hk, torch, tins, C, steps, warmup, 1, 1, prewarm_ms=pre, fa=fa, fb=fb)
        del tins
    flops, byts = 2.0 * M * N * K, algorithmic_bytes(M, N, K)
    out = {"M": M, "N": N, "K": K, "fmt_a": FMT_NAME[fa], "fmt_b": FMT_NAME[fb], "source_a": cfg["kind_a"], "source_b": cfg["kind_b"], "seed": cfg["seed"],
           "bound": cfg["bound"], "kernel_choice_row_major": hk.tk_kernel.kernel_choice(M, N, K, 0, 0),
           "row_major_ms": row_ms, "tile_major_ms": tile_ms, "algorithmic_flops": flops, "algorithmic_bytes": byts}
    best = min(t for t in (row_ms, tile_ms) if t is not None)
    if cfg["bound"] == "mfma":
        out.update({"row_major_tflops": flops / (row_ms * 1e-3) / 1e12, "tile_major_tflops": flops / (tile_ms * 1e-3) / 1e12 if tile_ms else None,
                    "frac_row_major": flops / (row_ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, "frac": flops / (best * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s"})
    else:
        out.update({"row_major_gbs": byts / (row_ms * 1e-3) / 1e9, "tile_major_gbs": byts / (tile_ms * 1e-3) / 1e9 if tile_ms else None,
                    "frac_row_major": byts / (row_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "frac": byts / (best * 1e-3) / 1e9 / HBM_PEAK_GBS, "peak": HBM_PEAK_GBS, "unit": "GB/s"})
    if cpu:
        # accuracy: 64 rows of A (all of A when it has fewer) over all of K, before the bf16 rounding
        rows = min(M, 64)
        k_slice = 8 if name in ("cfg2", "cfg4") else 1
        ap, bp, asc, bsc = ins[0]
        c32 = torch.empty(rows, N, dtype=torch.float32, device="cuda")
        hk.dispatch_micro(ap[:rows], bp, asc[:rows], bsc, c32, fa, fb)
        torch.cuda.synchronize()
        full = cpu_legs(cfg, ins[0], rows, 1, c32.cpu().numpy())
        out["max_rel_err"] = full["max_rel_err_gpu_vs_cpu"]
        out["max_rel_err_what"] = f"{rows} rows of the fp32 result over all of K against the CPU oracle; bar 2e-3"
        if k_slice == 1 and rows == M:
            out["cpu_baseline"] = full
        else:
            out["cpu_baseline"] = cpu_legs(cfg, ins[0], M if name != "cfg1" else M, k_slice, None)
    del ins, C
    torch.cuda.empty_cache()
    return out


def square_sizes(hk, torch, steps, warmup):
    """The other square sizes of the reference's published FP6 table: the operator from row-major inputs (whatever the
    library chooses, pre-pass included where it makes one) and on tile-major operands, back-to-back launches over
    three input sets (two at 16384); TFLOPS and the ratio to the published figure."""
    out = {"what": "M=N=K, e2m3 x e2m3, bf16 out: the operator on row-major inputs / on tile-major operands and scales; TFLOPS, and "
                   "over the reference's published MI355X FP6 figure for the size (analysis/fp6_gemm/mi355x_fp6_gemm.json)"}
    for S, ref in PUBLISHED_FP6_SQUARES.items():
        cfg = dict(M=S, N=S, K=S, fa=2, fb=2, kind_a="normal", kind_b="normal", seed=10 + S // 1024)
        ins = make_inputs(hk, torch, cfg, 2 if S > 8192 else 3)
        C = torch.empty(S, S, dtype=torch.bfloat16, device="cuda")
        pre = PREWARM_MS if S >= 4096 else 0.0
        _, row_ms = timed_loop(hk, torch, ins, C, steps, warmup, 0, 0, prewarm_ms=pre)
        tin = [tiled(hk, ops, S) for ops in ins]
        del ins
        _, tile_ms = timed_loop(hk, torch, tin, C, steps, warmup, 1, 1, prewarm_ms=pre)
        flops = 2.0 * S ** 3
        graph_ms = None
        if S <= 2048:
            # below ~10 us a launch the rate above is the host's: the same launches recorded into a graph (20 per
            # graph, tile-major operands) and replayed give the rate of the kernels themselves
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for i in range(20):
                    ap, bp, asc, bsc = tin[i % len(tin)]
                    hk.dispatch_micro(ap, bp, asc, bsc, C, layout_a=1, layout_b=1)
            for _ in range(3):
                graph.replay()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            for _ in range(10):
                graph.replay()
            e1.record()
            torch.cuda.synchronize()
            graph_ms = e0.elapsed_time(e1) / 200
            del graph
        out[str(S)] = {
            "row_major_ms": row_ms, "row_major_tflops": flops / (row_ms * 1e-3) / 1e12, "row_major_vs_published": flops / (row_ms * 1e-3) / 1e12 / ref,
            "tile_major_ms": tile_ms, "tile_major_tflops": flops / (tile_ms * 1e-3) / 1e12, "tile_major_vs_published": flops / (tile_ms * 1e-3) / 1e12 / ref,
            "kernel_choice_row_major": hk.tk_kernel.kernel_choice(S, S, S, 0, 0), "kernel_choice_tile_major": hk.tk_kernel.kernel_choice(S, S, S, 1, 1),
            "published_tflops": ref,
        }
        if graph_ms is not None:
            out[str(S)].update({"graph_replay_ms": graph_ms, "graph_replay_tflops": flops / (graph_ms * 1e-3) / 1e12})
        del tin, C
        torch.cuda.empty_cache()
    return out


def weight_sets(hk, torch, N, K, gen):
    """A weight matrix [N, K] in as many rotated copies as make 400 MB (2 to 16), row-major and tile-major, each kind in one
    contiguous buffer: the timing probe takes launch i's weights from copy i % sets, so that B comes from HBM as the weights
    of a model's layers do, not from the 256 MB last-level cache."""
    b, sc = hk.quantize(torch.randn(N, K, device="cuda", generator=gen) * 0.02, 2)
    sets = min(16, max(2, -(-400_000_000 // (N * K * 3 // 4))))
    bp = torch.stack([torch.roll(b, 32 * i, 0) for i in range(sets)])
    bs = torch.stack([torch.roll(sc, 32 * i, 0) for i in range(sets)])
    del b, sc
    bt = torch.stack([hk.tile_operand(bp[i]) for i in range(sets)])
    bst = torch.stack([hk.tile_scales(bs[i], K) for i in range(sets)])
    return sets, (bp, bs), (bt, bst)


def probe_time_us(P, torch, a, asc, weights, sets, C, M, N, K, la, lb, kernel, k_split):
    """Microseconds per launch of one GEMM with a kernel forced (0: the automatic choice) and a K-split setting, timed by the
    measurement build between two events around back-to-back launches (mxfp6_probe_time_gemm: no interpreter between the
    launches, so a shape of a few microseconds is timed as a replayed graph would run it); None: the forced kernel does not
    take the shape.  A first short run sizes the timed one to about 0.6 ms."""
    import ctypes

    B, Bs = weights
    stream = torch.cuda.current_stream().cuda_stream
    us = ctypes.c_double()
    prev_k, prev_s = P.mxfp6_set_kernel(kernel), P.mxfp6_set_k_split(k_split)
    try:
        def run(warmup, reps):
            return P.mxfp6_probe_time_gemm(a.data_ptr(), B.data_ptr(), asc.data_ptr(), Bs.data_ptr(), C.data_ptr(), M, N, K, 2, 2, la, lb, 0, sets,
                                           B.stride(0) * B.element_size(), Bs.stride(0) * Bs.element_size(), warmup, reps, ctypes.byref(us), stream)
        if run(2, 4) != 0:
            return None
        if run(2, max(8, min(64, int(600.0 / max(us.value, 1.0))))) != 0:
            return None
    finally:
        P.mxfp6_set_kernel(prev_k)
        P.mxfp6_set_k_split(prev_s)
    return us.value


CANDIDATES = (("tiled_256x256", 6, 1), ("tiled_128x256", 5, 1), ("tiled_128x128", 17, 1), ("block", 22, 1), ("block_128x256", 26, 1), ("skinny", 3, 0),
              ("tiled_k_split_256", 6, -1), ("tiled_k_split_128", 5, -1), ("block_k_split", 22, -1), ("ring", 28, 0))  # in the order of the library's candidate numbers


def dispatch_sweep(hk, torch, grid):
    """How good is the automatic kernel choice?  For every shape of a grid (rows of A x a set of (N, K) pairs x both
    layouts of B; A row-major) the call is timed with the automatic choice (twice, before and after the others: the better
    of the two) and with every kernel / tile shape forced in turn, the tiled and the block kernel also with their K split
    wherever the shape allows one.  Reports, per shape, the automatic time, the best forced time and which kernel that was,
    and the shapes where the automatic choice is more than 8 % behind.  Timed on the GPU's side (probe_time_us), weights
    rotating through 400 MB."""
    from hipkittensp_amd import _lib

    tk, P = hk.tk_kernel, _lib.probes()
    if grid == "offgrid":  # none of these (N, K) pairs and none of these row counts is in the calibration table
        shapes = [(7168, 7168), (3584, 18944), (18944, 3584), (9216, 4608), (27648, 5120), (1792, 14336), (22016, 4096), (5632, 22528),
                  (13312, 6656), (36864, 3072), (2304, 24576), (15360, 10240)]
        rows_of_a = [20, 56, 72, 144, 208, 288, 416, 576, 832, 1152, 1792, 2560]
    elif grid == "offgrid2":  # a second held-out set, never used to tune anything
        shapes = [(5120, 5120), (9216, 9216), (14336, 7168), (3328, 16640), (25600, 5632), (2816, 11264), (45056, 3584), (6656, 13312),
                  (19456, 6144), (1280, 28160), (10752, 10752), (30720, 2560)]
        rows_of_a = [28, 36, 88, 104, 176, 240, 352, 480, 704, 960, 1280, 2304]
    elif grid == "full":
        shapes = [(8192, 8192), (4096, 14336), (28672, 8192), (28672, 4096), (24576, 8192), (40960, 8192), (57344, 8192), (128256, 4096),
                  (8192, 28672), (2048, 8192), (5120, 16384), (10240, 8192), (1024, 16384), (14336, 4096), (32000, 4096)]
        rows_of_a = [8, 16, 24, 32, 48, 64, 96, 128, 192, 256, 384, 512, 768, 1024, 2048]
    else:
        shapes = [(8192, 8192), (28672, 8192), (8192, 28672), (57344, 8192), (1024, 16384)]
        rows_of_a = [16, 32, 64, 128, 256, 512, 1024]
    forced = (("tiled", 2, 1), ("mid", 4, 0)) + CANDIDATES

    per_shape, behind = [], []
    g = torch.Generator(device="cuda")
    g.manual_seed(1)
    for N, K in shapes:
        sets, row, tile = weight_sets(hk, torch, N, K, g)
        for M in rows_of_a:
            a, asc = hk.quantize(torch.randn(M, K, device="cuda", generator=g), 2)
            C = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
            for lay in (1, 0):
                def t(kernel, k_split):
                    return probe_time_us(P, torch, a, asc, tile if lay else row, sets, C, M, N, K, 0, lay, kernel, k_split)
                auto = t(0, 0)
                times = {}
                for name, kernel, k_split in forced:
                    if (name == "skinny" and M > 128) or (name == "mid" and (M <= 32 or M > 512)) or (name == "ring" and M > 256):
                        continue
                    us = t(kernel, k_split)
                    if us is not None:
                        times[name] = us
                auto = min(auto, t(0, 0))
                best = min(times, key=times.get)
                rec = {"M": M, "N": N, "K": K, "layout_b": "tile" if lay else "row", "auto_us": round(auto, 2), "best_us": round(times[best], 2),
                       "best": best, "auto_over_best": round(auto / times[best], 3), "times_us": {k: round(v, 2) for k, v in times.items()},
                       "choice": tk.kernel_choice(M, N, K, 0, lay)}
                per_shape.append(rec)
                if rec["auto_over_best"] > 1.08:
                    behind.append(rec)
        del row, tile
        torch.cuda.empty_cache()
    ratios = sorted(r["auto_over_best"] for r in per_shape)
    return {"what": "automatic kernel choice against every forced kernel, tile shape and K split; e2m3 x e2m3, bf16 out, A row-major; timed on the GPU's side, weights rotating through 400 MB",
            "shapes": len(per_shape), "within_8_percent": sum(1 for r in ratios if r <= 1.08), "median_auto_over_best": ratios[len(ratios) // 2], "worst_auto_over_best": ratios[-1],
            "behind_by_more_than_8_percent": behind, "per_shape": per_shape}


def calibration_sweep(hk, torch):
    """The sweep behind the kernel choice's calibration table (hipkittensp_amd/csrc/dispatch_table.inc): every candidate of the
    choice, forced, on a grid of shapes x three layout pairs, timed on the GPU's side with weights rotating through 400 MB
    (probe_time_us), twice (the better counts).  `python -m hipkittensp_amd.calibrate` turns the JSON this prints into the
    table: per shape and candidate, measured time / the time model's figure."""
    import ctypes

    from hipkittensp_amd import _lib

    tk, P = hk.tk_kernel, _lib.probes()
    shapes = [(8192, 8192), (4096, 14336), (28672, 8192), (28672, 4096), (24576, 8192), (40960, 8192), (57344, 8192), (128256, 4096), (8192, 28672), (2048, 8192), (5120, 16384),
              (10240, 8192), (1024, 16384), (14336, 4096), (32000, 4096), (4096, 4096), (16384, 16384), (2048, 28672), (11008, 4096), (4096, 11008), (2048, 2048), (512, 8192), (8192, 1024),
              (1024, 32768), (2048, 16384), (4096, 8192), (4096, 24576), (8192, 4096), (8192, 14336), (16384, 4096), (16384, 8192), (65536, 2048), (3072, 3072), (6144, 4096), (1024, 4096),
              (12288, 12288), (2048, 5120), (24576, 2048), (73728, 4096),
              (6144, 6144), (12288, 6144), (3072, 12288), (20480, 5120), (18432, 9216), (7168, 20480), (49152, 4096), (2560, 10240), (13824, 5120), (5120, 13824), (100352, 2048), (1536, 32768)]
    rows_of_a = [1, 8, 12, 16, 24, 32, 40, 48, 64, 80, 96, 112, 128, 160, 192, 224, 256, 320, 384, 448, 512, 640, 768, 896, 1024, 1536, 2048, 3072, 4096, 8192]

    points = []
    g = torch.Generator(device="cuda")
    g.manual_seed(1)
    for N, K in shapes:
        sets, row, tile = weight_sets(hk, torch, N, K, g)
        for M in rows_of_a:
            if M * N > 1 << 28:
                continue
            a, asc = hk.quantize(torch.randn(M, K, device="cuda", generator=g), 2)
            C = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
            for la, lb in ((0, 0), (0, 1), (1, 1)):
                if la and (M % 32 or K % 128):
                    continue
                at, ast = (hk.tile_operand(a), hk.tile_scales(asc, K)) if la else (a, asc)
                layouts = la | lb << 1

                def t(kernel, k_split):
                    return probe_time_us(P, torch, at, ast, tile if lb else row, sets, C, M, N, K, la, lb, kernel, k_split)
                measured = []
                for cand, (name, kernel, k_split) in enumerate(CANDIDATES):
                    m, c, sh = ctypes.c_double(), ctypes.c_double(), ctypes.c_int()
                    prev = P.mxfp6_set_k_split(k_split)
                    rc = P.mxfp6_probe_candidate(M, N, K, layouts, cand, 0, ctypes.byref(m), ctypes.byref(c), ctypes.byref(sh))
                    P.mxfp6_set_k_split(prev)
                    assert rc == 0, rc
                    us = None
                    if m.value >= 0:  # the candidate takes the shape (a split: the shape has one)
                        us = t(kernel, k_split)
                        us2 = t(kernel, k_split) if us is not None else None
                        us = min(us, us2) if us2 is not None else us
                    measured.append(round(us, 2) if us is not None else None)
                point = {"M": M, "N": N, "K": K, "layouts": layouts, "measured_us": measured, "auto_us": round(t(0, 0), 2), "choice": tk.kernel_choice(M, N, K, la, lb)}
                if measured[-1] is not None:  # the ring kernel as one share of K: not a candidate of its own, a point for the model's per-workgroup rate
                    one = t(CANDIDATES[-1][1], 1)
                    point["ring_one_share_us"] = round(one, 2) if one is not None else None
                points.append(point)
        del row, tile
        torch.cuda.empty_cache()
    return {"what": "calibration sweep of the kernel choice: measured microseconds per candidate (GPU-side timing, weights rotating through 400 MB)", "candidates": [c[0] for c in CANDIDATES],
            "device": torch.cuda.get_device_name(0), "cus": torch.cuda.get_device_properties(0).multi_processor_count, "points": points}


def source_hash(kernel):
    h = hashlib.sha256()
    for f in TRAFFIC_SOURCES[kernel]:
        h.update(open(os.path.join(ROOT, "hipkittensp_amd", "csrc", f), "rb").read())
    return h.hexdigest()[:16]


def traffic_of(kernel):
    """Fabric bytes per launch of a kernel, from profiles/traffic.json (written by `bench.py --traffic-from`, from two
    rocprofv3 --pmc runs of this file).  The kernels move the same bytes on every launch of a shape, but only as long as
    their source is what was profiled: the entry carries the hash of the kernel's sources, and a stale entry gives null."""
    try:
        rec = json.load(open(TRAFFIC_JSON))["kernels"][kernel]
    except (OSError, KeyError, ValueError):
        return None, "profiles/traffic.json has no entry for this kernel"
    if rec.get("source_hash") != source_hash(kernel):
        return None, "profiles/traffic.json was taken on other kernel sources (hash mismatch): re-profile"
    return rec["traffic_bytes"], rec.get("what", "")


def traffic_from(fetch_csv, write_csv):
    """Reads the counter_collection CSVs of `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` runs of `bench.py
    --profile-kernels` and writes profiles/traffic.json.  Calibration inside the same runs: a copy of known size (torch's
    in-place x *= 0.02 on 8192 x 28672 fp32: 917 504 KiB read and written) fixes what one count is worth."""
    import collections
    import csv
    import re

    def per_kernel(path):
        agg = collections.defaultdict(list)
        for r in csv.DictReader(open(path)):
            agg[re.sub(r"\(.*$", "", re.sub(r"^void ", "", r["Kernel_Name"].replace("(anonymous namespace)::", "")))].append(float(r["Counter_Value"]))
        return agg

    fetch, write = per_kernel(fetch_csv), per_kernel(write_csv)
    known_kib = 8192 * 28672 * 4 / 1024.0

    def calib(agg):
        vals = [max(v) for k, v in agg.items() if "elementwise" in k.lower() and max(v) > 1e5]
        assert vals, "calibration kernel not found in the trace"
        return known_kib / max(vals)

    ff, wf = calib(fetch), calib(write)
    out = {"what": "FETCH_SIZE and WRITE_SIZE (KiB per dispatch) of rocprofv3 --pmc runs of `python3 bench.py --profile-kernels`, each scaled by what the same "
                   "counter reads for an elementwise in-place multiply of 8192 x 28672 fp32 (917 504 KiB each way) in the same run",
           "fetch_factor": ff, "write_factor": wf, "kernels": {}}
    for kernel, match in (("gemm_tiled_kernel", "gemm_tiled_kernel<2, 2, mxfp6::OutBf16, 4, 2"), ("gemm_skinny_kernel", "gemm_skinny_kernel<2, 2, mxfp6::OutBf16, 16, 8, 32"),
                          ("gemm_ring_kernel_m16", "gemm_ring_kernel<2, 2, mxfp6::OutBf16, 1>"), ("gemm_ring_kernel_m64", "gemm_ring_kernel<2, 2, mxfp6::OutBf16, 2>")):
        f = [max(v) for k, v in fetch.items() if match in k]
        w = [max(v) for k, v in write.items() if match in k]
        if not (f and w):   # the decode loop ran on the other of the two kernels that are level at configs[3]
            assert "tiled" not in kernel, f"{kernel} not found in the traces"
            continue
        out["kernels"][kernel] = {"fetch_kib": max(f), "write_kib": max(w), "traffic_bytes": int((max(f) * ff + max(w) * wf) * 1024), "source_hash": source_hash(kernel),
                                  "what": f"FETCH_SIZE {max(f):.0f} KiB x {ff:.2f} + WRITE_SIZE {max(w):.0f} KiB x {wf:.2f}"}
    json.dump(out, open(TRAFFIC_JSON, "w"), indent=1)
    print(json.dumps(out))


def main():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=100)
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--cpu-rows", type=int, default=8192)
    p.add_argument("--raster-sweep", action="store_true", help="only time the tiled kernel at 8192^3 (tile-major operands) over raster settings and print one JSON line")
    p.add_argument("--kernel", type=int, default=0, help="with --raster-sweep: kernel code to time as well (18 = the 4-wave schedule)")
    p.add_argument("--shape", type=int, nargs=3, metavar=("M", "N", "K"), default=None, help="with --raster-sweep: the problem shape (default 8192 8192 8192)")
    p.add_argument("--sweep-settings", choices=["all", "default", "ksplit-order"], default="all",
                   help="with --raster-sweep: all raster settings, only the kernel's own (to compare schedules under a profiler), or the kernel's own and, as "
                        "xcd_remap=2, a K split's workgroups in tile-by-tile order instead of share by share (for shapes that take a K split)")
    p.add_argument("--dispatch-sweep", choices=["small", "full", "offgrid", "offgrid2", "calibrate"], default=None,
                   help="only compare the automatic kernel choice with every forced kernel / tile shape / K split over a grid of shapes and print one JSON line")
    p.add_argument("--layouts", choices=["both", "row"], default="both", help="row: skip the decode run with tile-major weights (used for profiling one layout of the skinny kernel)")
    p.add_argument("--profile-kernels", action="store_true", help="only loops of the tiled kernel (8192^3, tile-major), the skinny kernel (configs[3], row-major) and the ring "
                                                                  "kernel (M = 64, tile-major weights), and a copy of known size: the run to put under rocprofv3 "
                                                                  "(--kernel-trace --stats, or --pmc FETCH_SIZE / WRITE_SIZE with --steps 5 --warmup 2)")
    p.add_argument("--traffic-from", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"), default=None,
                   help="no GPU: read the two counter_collection CSVs of --profile-kernels runs and write profiles/traffic.json")
    args = p.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures ONE GPU (a single-GPU operator; sharding is by N or M with no exchange). Run with --gpus 1.")
    if args.traffic_from:
        traffic_from(*args.traffic_from)
        return

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    import hipkittensp_amd as hk
    from hipkittensp_amd import _lib

    _lib.lib()  # fail loudly if the HIP library is missing
    tk = hk.tk_kernel

    if args.dispatch_sweep == "calibrate":
        print(json.dumps(calibration_sweep(hk, torch)))
        return
    if args.dispatch_sweep:
        print(json.dumps(dispatch_sweep(hk, torch, args.dispatch_sweep)))
        return

    cfg1 = CONFIGS["cfg1"]
    if args.profile_kernels:
        # the three kernels the profiles/ summaries are about, each in a loop of its own, and a copy of known size
        out = {"what": "per-launch milliseconds by device events; the rocprofv3 kernel trace of this run must agree", "steps": args.steps, "warmup": args.warmup}
        ins = make_inputs(hk, torch, cfg1, 2)
        kin = [tiled(hk, ops, cfg1["K"]) for ops in ins]
        del ins
        C = torch.empty(8192, 8192, dtype=torch.bfloat16, device="cuda")
        out["gemm_tiled_kernel_8192_cubed_tile_major_ms"] = timed_loop(hk, torch, kin, C, args.steps, args.warmup, 1, 1, prewarm_ms=PREWARM_MS)[1]
        del kin, C
        cfg3 = CONFIGS["cfg3"]
        d = make_inputs(hk, torch, cfg3, 5)
        dC = torch.empty(16, 8192, dtype=torch.bfloat16, device="cuda")
        for name, code in (("gemm_skinny_kernel", tk.KERNEL_SKINNY), ("gemm_ring_kernel", tk.KERNEL_RING)):  # level with each other at configs[3]: both
            prev = tk.set_kernel(code)
            try:
                out[name + "_cfg3_row_major_ms"] = timed_loop(hk, torch, d, dC, args.steps, args.warmup)[1]
            finally:
                tk.set_kernel(prev)
        out["cfg3_row_major_automatic_choice"] = DECODE_KERNELS.get(tk.kernel_choice(16, 8192, cfg3["K"], 0, 0), "?")
        dt = [tiled(hk, ops, cfg3["K"], "b") for ops in d]
        del d
        ba, bas = hk.quantize(torch.from_numpy(cpu_source("normal", (64, cfg3["K"]), 3164)).cuda(), 2)
        bC = torch.empty(64, 8192, dtype=torch.bfloat16, device="cuda")
        out["gemm_ring_kernel_m64_tile_major_weights_ms"] = timed_loop(hk, torch, [(ba, bt, bas, bst) for _, bt, _, bst in dt], bC, args.steps, args.warmup, 0, 1)[1]
        x = torch.ones(8192, 28672, device="cuda")
        x *= 0.02
        torch.cuda.synchronize()
        print(json.dumps(out))
        return

    # ---- headline: configs[1], 8192^3 e2m3 x e2m3 -> bf16
    M, N, K = cfg1["M"], cfg1["N"], cfg1["K"]
    if args.raster_sweep and args.shape:
        M, N, K = args.shape
    inputs = make_inputs(hk, torch, dict(cfg1, M=M, N=N, K=K), 3 if not (args.raster_sweep and args.shape) else 2)
    C = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    if args.raster_sweep:
        # the tiled kernel alone on tile-major operands, per raster setting (the kernel's own: 4 tile rows per group, XCD remap on);
        # through the measurement build, which has the override
        P = _lib.probes()
        stream = torch.cuda.current_stream().cuda_stream
        P.mxfp6_set_relayout(0)
        kin = [tiled(hk, ops, K) for ops in inputs]

        def call(ops):
            rc = P.mxfp6_gemm_ex(ops[0].data_ptr(), ops[1].data_ptr(), ops[2].data_ptr(), ops[3].data_ptr(), C.data_ptr(), M, N, K, 2, 2, 1, 1, 0, stream)
            assert rc == 0, rc
        res = {}
        for rnd in range(2):  # two rounds over all settings: the second is reported (the first also warms the chip up)
            for xcd in {"all": (1, 0), "default": (1,), "ksplit-order": (1, 2)}[args.sweep_settings]:
                for gm in ((1, 2, 4, 8, 16, 32) if args.sweep_settings == "all" else (4,)):
                    assert P.mxfp6_probe_raster(gm, xcd) == 0
                    _, ms = timed_loop(hk, torch, kin, C, args.steps, args.warmup, call=call)
                    res[f"xcd_remap={xcd},group_m={gm}"] = {"launch_ms_mean": ms, "tflops": 2.0 * M * N * K / (ms * 1e-3) / 1e12}
            P.mxfp6_probe_raster(0, 1)
            if args.kernel:
                prevk = P.mxfp6_set_kernel(args.kernel)
                _, ms = timed_loop(hk, torch, kin, C, args.steps, args.warmup, call=call)
                P.mxfp6_set_kernel(prevk)
                res[f"kernel={args.kernel}"] = {"launch_ms_mean": ms, "tflops": 2.0 * M * N * K / (ms * 1e-3) / 1e12}
        print(json.dumps({"what": f"the kernel the library chooses ({tk.kernel_choice(M, N, K, 1, 1)}: 2 = gemm_tiled_kernel, 22 = gemm_block_kernel, 25 = tiled with K split), {M} x {N} x {K} e2m3, operands and scales tile-major, per raster setting", "steps": args.steps, "warmup": args.warmup, "settings": res}))
        return
    # the operator as a caller gets it: for this size the library re-lays both operands out tile-major in a
    # pre-pass (one small kernel for both) and runs the tiled kernel on them; `value` is the whole step
    wall, step_ms = timed_loop(hk, torch, inputs, C, args.steps, args.warmup, prewarm_ms=PREWARM_MS)
    flops = 2.0 * M * N * K
    ms_per_step = wall / args.steps * 1e3
    value = flops / (wall / args.steps) / 1e12
    # weights prepared once (B and its scales tile-major: mxfp6_blob_pack / tile_operand at load time), activations
    # row-major as they come: the pre-pass copies A only
    pinputs = [tiled(hk, ops, K, "b") for ops in inputs]
    pwall, pstep_ms = timed_loop(hk, torch, pinputs, C, args.steps, args.warmup, 0, 1, prewarm_ms=PREWARM_MS)
    del pinputs
    # the dominant kernel by itself, in the configuration the step launches it in (both operands tile-major):
    # the same inputs re-laid out beforehand, pre-pass off
    prev = tk.set_relayout(False)
    kinputs = [tiled(hk, ops, K) for ops in inputs]
    _, ev_ms = timed_loop(hk, torch, kinputs, C, args.steps, args.warmup, 1, 1, prewarm_ms=PREWARM_MS)
    # and the tiled kernel on the row-major operands themselves (what the pre-pass avoids)
    _, row_ms = timed_loop(hk, torch, inputs, C, args.steps, args.warmup, prewarm_ms=PREWARM_MS)
    tk.set_relayout(prev)
    sustained = probes(hk, torch, _lib.probes(), inputs, kinputs, C, M, N, K)
    del kinputs
    ref_protocol = per_launch_ref_protocol(hk, torch, M, N, K, 20, seed=11)
    achieved = flops / (ev_ms * 1e-3) / 1e12
    traffic, traffic_what = traffic_of("gemm_tiled_kernel")
    # the matrix cores' own ceiling on these operand bits: the higher of the MFMA-only probe and the kernel's MFMA-only build
    mfma_ceiling = max(sustained["mfma_only_real_operands"]["tflops"], sustained["mfma_only_build_tflops"])
    roofline = {
        "kernel": "gemm_tiled_kernel (256x256x128 tiles, v_mfma_scale_f32_32x32x64_f8f6f4) on the tile-major copies the pre-pass makes of both operands",
        "bound": "mfma",
        "achieved": achieved,
        "peak": MFMA_PEAK_TFLOPS,
        "unit": "TFLOP/s",
        "frac": achieved / MFMA_PEAK_TFLOPS,
        "traffic": traffic,
        "traffic_what": traffic_what,
        "launch_ms_mean": ev_ms,
        "step_ms_mean": step_ms,
        "prepass_ms_mean": step_ms - ev_ms,
        "prepass_a_only_ms_mean": pstep_ms - ev_ms,
        "algorithmic_flops_per_launch": flops,
        "algorithmic_bytes_per_launch": algorithmic_bytes(M, N, K),
        "hbm_bound_ms": algorithmic_bytes(M, N, K) / (HBM_PEAK_GBS * 1e9) * 1e3,
        "sustained_mfma_tflops": mfma_ceiling,
        "frac_of_sustained_mfma": achieved / mfma_ceiling,
        "sustained": sustained,
        "per_launch_ms_ref_protocol": ref_protocol["kernel_tile_major_ms_median"],
        "ref_protocol": ref_protocol,
        "row_major_kernel": {"what": "gemm_tiled_kernel on both operands row-major (pre-pass off)", "launch_ms_mean": row_ms,
                             "achieved": flops / (row_ms * 1e-3) / 1e12, "frac": flops / (row_ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS},
    }

    cpu = None
    configs = {}
    if not args.no_cpu_baseline:
        c32 = torch.empty(args.cpu_rows, N, dtype=torch.float32, device="cuda")
        ap0, bp0, asc0, bsc0 = inputs[0]
        hk.dispatch_micro(ap0[: args.cpu_rows], bp0, asc0[: args.cpu_rows], bsc0, c32)
        torch.cuda.synchronize()
        gpu_f32 = c32.cpu().numpy()
        del c32
        legs = cpu_legs(cfg1, inputs[0], args.cpu_rows, 1, gpu_f32)
        del gpu_f32
        cpu = dict(legs["port"], max_rel_err_gpu_vs_cpu=legs["max_rel_err_gpu_vs_cpu"], max_rel_err_bar=2e-3, sample=legs["sample"] + ", one pass", torch_matmul=legs["torch_matmul"])
    configs["cfg1"] = {"M": M, "N": N, "K": K, "fmt_a": "e2m3", "fmt_b": "e2m3", "source_a": "normal", "source_b": "normal", "seed": 1, "bound": "mfma",
                       "row_major_ms": step_ms, "row_major_tflops": flops / (step_ms * 1e-3) / 1e12, "tile_major_ms": ev_ms, "tile_major_tflops": achieved,
                       "frac_row_major": flops / (step_ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, "frac": achieved / MFMA_PEAK_TFLOPS, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                       "max_rel_err": cpu["max_rel_err_gpu_vs_cpu"] if cpu else None, "max_rel_err_what": "all of the fp32 result against the CPU oracle; bar 2e-3",
                       "cpu_baseline": {"port": {k: cpu[k] for k in ("value", "unit", "seconds", "cores", "kind")}, "torch_matmul": cpu["torch_matmul"], "sample": cpu["sample"], "k_slice": 1} if cpu else None}

    # callers that keep their operands tile-major (MXFP6_LAYOUT_TILE; weights converted once, activations straight
    # from the quantiser) skip the pre-pass: that is the kernel-only figure above
    tile_major = {
        "what": "same 8192^3 workload, operands and scales already tile-major (mxfp6_tile_operand + mxfp6_tile_scales / quantiser output): no pre-pass",
        "value": achieved, "unit": "TFLOPS", "achieved": achieved, "frac": achieved / MFMA_PEAK_TFLOPS, "launch_ms_mean": ev_ms,
    }
    del inputs
    del C
    torch.cuda.empty_cache()

    # ---- the other configurations, each with its own distributions and formats
    for name in ("cfg0", "cfg2", "cfg4"):
        configs[name] = run_config(hk, torch, name, args.steps, args.warmup, not args.no_cpu_baseline)

    # ---- decode shape: configs[3], M=16, N=8192, K=28672, weights N(0, 0.02); five weight sets
    # (5 x 184 MB > the 256 MB last-level cache) so that the rate is HBM's, not the cache's
    cfg3 = CONFIGS["cfg3"]
    dM, dN, dK = cfg3["M"], cfg3["N"], cfg3["K"]
    dinputs = make_inputs(hk, torch, cfg3, 5)
    dC = torch.empty(dM, dN, dtype=torch.bfloat16, device="cuda")
    dwall, dev_ms = timed_loop(hk, torch, dinputs, dC, args.steps, args.warmup)
    dbytes = algorithmic_bytes(dM, dN, dK)
    d_achieved = dbytes / (dev_ms * 1e-3) / 1e9
    dtile = dbatched = dmid = dprefill = dm32 = None
    cfg3_entry = {"M": dM, "N": dN, "K": dK, "fmt_a": "e2m3", "fmt_b": "e2m3", "source_a": "normal", "source_b": "weights", "seed": 3, "bound": "hbm",
                  "kernel_choice_row_major": tk.kernel_choice(dM, dN, dK, 0, 0), "row_major_ms": dev_ms, "row_major_gbs": d_achieved, "frac_row_major": d_achieved / HBM_PEAK_GBS,
                  "algorithmic_bytes": dbytes, "algorithmic_flops": 2.0 * dM * dN * dK, "peak": HBM_PEAK_GBS, "unit": "GB/s"}
    if not args.no_cpu_baseline:
        c32 = torch.empty(dM, dN, dtype=torch.float32, device="cuda")
        hk.dispatch_micro(dinputs[0][0], dinputs[0][1], dinputs[0][2], dinputs[0][3], c32)
        torch.cuda.synchronize()
        legs = cpu_legs(cfg3, dinputs[0], dM, 1, c32.cpu().numpy())
        cfg3_entry.update({"max_rel_err": legs["max_rel_err_gpu_vs_cpu"], "max_rel_err_what": "all of the fp32 result against the CPU oracle; bar 2e-3", "cpu_baseline": legs})
    if args.layouts == "both":
        dtin = [tiled(hk, ops, dK, "b") for ops in dinputs]
        dtwall, dtev_ms = timed_loop(hk, torch, dtin, dC, args.steps, args.warmup, 0, 1)
        cfg3_entry.update({"tile_major_ms": dtev_ms, "tile_major_gbs": dbytes / (dtev_ms * 1e-3) / 1e9, "frac": dbytes / (min(dtev_ms, dev_ms) * 1e-3) / 1e9 / HBM_PEAK_GBS})

        def batched(bM, la):
            x = torch.from_numpy(cpu_source("normal", (bM, dK), 3100 + bM)).cuda()
            ba, bas = hk.quantize(x, 2, layout=hk.LAYOUT_TILE if la else hk.LAYOUT_ROW)
            bC = torch.empty(bM, dN, dtype=torch.bfloat16, device="cuda")
            ins = [(ba, bt, bas, bst) for _, bt, _, bst in dtin]
            _, ms = timed_loop(hk, torch, ins, bC, args.steps, args.warmup, la, 1)
            byts = algorithmic_bytes(bM, dN, dK)
            return ins, bC, ms, byts
        # batched decode: 32 and 64 rows of a row-major A against the same tile-major weights
        _, _, m32_ms, m32_bytes = batched(32, 0)
        dm32 = {"what": "M=32 (row-major A) against the same tile-major weights", "kernel_choice": tk.kernel_choice(32, dN, dK, 0, 1), "achieved": m32_bytes / (m32_ms * 1e-3) / 1e9,
                "unit": "GB/s", "frac": m32_bytes / (m32_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "launch_ms_mean": m32_ms, "algorithmic_bytes_per_launch": m32_bytes}
        _, _, bev_ms, bbytes = batched(64, 0)
        dbatched = {
            "what": "M=64 (row-major A) against the same tile-major weights (kernel_choice 3: gemm_skinny_kernel, 28: gemm_ring_kernel, 25 / 27: gemm_tiled_kernel / gemm_block_kernel with K split between workgroups)",
            "kernel_choice": tk.kernel_choice(64, dN, dK, 0, 1), "achieved": bbytes / (bev_ms * 1e-3) / 1e9, "unit": "GB/s",
            "frac": bbytes / (bev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "launch_ms_mean": bev_ms, "algorithmic_bytes_per_launch": bbytes,
        }
        # a few hundred rows of A against the same weights: a K split between workgroups, and the best kernel without one
        mins, mC, mev_ms, mbytes = batched(256, 1)
        prev_split = tk.set_k_split(1)
        try:
            _, mev_ms_unsplit = timed_loop(hk, torch, mins, mC, args.steps, args.warmup, 1, 1)
        finally:
            tk.set_k_split(prev_split)
        mflops = 2.0 * 256 * dN * dK
        dmid = {
            "what": "M=256 against the same tile-major weights (A tile-major too): K split between workgroups (kernel_choice 25: gemm_tiled_kernel, 27: gemm_block_kernel) + ksplit_reduce_kernel",
            "kernel_choice": tk.kernel_choice(256, dN, dK, 1, 1), "launch_ms_mean": mev_ms, "achieved": mbytes / (mev_ms * 1e-3) / 1e9,
            "unit": "GB/s", "frac": mbytes / (mev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "tflops": mflops / (mev_ms * 1e-3) / 1e12,
            "launch_ms_mean_without_split": mev_ms_unsplit, "algorithmic_bytes_per_launch": mbytes,
        }
        del dtin, mins
        # a few hundred rows of A at a K that is too short to split: gemm_block_kernel (128 x 128 tiles, four waves in
        # step) against the 8-wave tiled kernel's 128 x 128 tiles, both operands tile-major
        pM, pN, pK = 512, 8192, 8192
        pcfg = dict(M=pM, N=pN, K=pK, fa=2, fb=2, kind_a="normal", kind_b="weights", seed=7)
        pins = [tiled(hk, ops, pK) for ops in make_inputs(hk, torch, pcfg, 3)]
        pC = torch.empty(pM, pN, dtype=torch.bfloat16, device="cuda")
        _, pev_ms = timed_loop(hk, torch, pins, pC, args.steps, args.warmup, 1, 1)
        prevk = tk.set_kernel(tk.KERNEL_TILED_128x128)
        try:
            _, pev_ms_tiled = timed_loop(hk, torch, pins, pC, args.steps, args.warmup, 1, 1)
        finally:
            tk.set_kernel(prevk)
        dprefill = {
            "what": "M=512, N=K=8192, operands tile-major: the automatic choice (gemm_block_kernel) and the 8-wave tiled kernel with the same 128 x 128 tiles",
            "kernel_choice": tk.kernel_choice(pM, pN, pK, 1, 1), "launch_ms_mean": pev_ms, "tflops": 2.0 * pM * pN * pK / (pev_ms * 1e-3) / 1e12,
            "launch_ms_mean_tiled_128x128": pev_ms_tiled,
        }
        del pins, pC
        dtile = {
            "what": "same decode workload, weights (B) and their scales tile-major",
            "achieved": dbytes / (dtev_ms * 1e-3) / 1e9, "unit": "GB/s", "frac": dbytes / (dtev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "launch_ms_mean": dtev_ms,
        }
    configs["cfg3"] = cfg3_entry
    configs = {k: configs[k] for k in sorted(configs)}
    del dinputs
    torch.cuda.empty_cache()
    squares = square_sizes(hk, torch, args.steps, args.warmup) if args.layouts == "both" else None
    # ---- the quantiser (the step in front of the GEMM at inference time): 8192 x 8192 activations -> packed fp6 + E8M0,
    # fp32 and bf16 sources, into preallocated outputs through the C ABI (no allocation inside the timed region)
    torch.cuda.empty_cache()
    L = _lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    quant = {"what": "fp32 / bf16 [8192, 8192] -> packed e2m3 + E8M0 scales (row-major), bytes read + written per launch", "bound": "hbm",
             "peak": HBM_PEAK_GBS, "unit": "GB/s"}
    q0 = torch.from_numpy(cpu_source("normal", (8192, 8192), 21)).cuda()
    qx = [q0, torch.roll(q0, 1, 0), torch.roll(q0, 2, 0)]
    qp = torch.empty(8192, 6144, dtype=torch.uint8, device="cuda")
    qs = torch.empty(8192, 256, dtype=torch.uint8, device="cuda")
    for name, fn, xs in (("fp32", L.mxfp6_quantize_ex, qx), ("bf16", L.mxfp6_quantize_bf16, [x.to(torch.bfloat16) for x in qx])):
        for i in range(args.warmup):
            fn(xs[i % 3].data_ptr(), qp.data_ptr(), qs.data_ptr(), 8192, 8192, 2, 0, stream)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for i in range(args.steps):
            rc = fn(xs[i % 3].data_ptr(), qp.data_ptr(), qs.data_ptr(), 8192, 8192, 2, 0, stream)
        e1.record()
        torch.cuda.synchronize()
        assert rc == 0
        ms = e0.elapsed_time(e1) / args.steps
        qbytes = 8192 * 8192 * (xs[0].element_size() + 0.75 + 1 / 32)
        quant[name] = {"launch_ms_mean": ms, "achieved": qbytes / (ms * 1e-3) / 1e9, "frac": qbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                       "algorithmic_bytes_per_launch": qbytes}
    del qx, qp, qs, q0
    torch.cuda.empty_cache()
    stream_p = stream_probe(torch, _lib.probes())
    dkernel = DECODE_KERNELS.get(tk.kernel_choice(dM, dN, dK, 0, 0), "?")  # the skinny and the ring kernel are level here
    dtraffic, dtraffic_what = traffic_of("gemm_ring_kernel_m16" if dkernel == "gemm_ring_kernel" else dkernel)
    decode = {
        "metric": "MXFP6 decode GEMM achieved GB/s @M=16,N=8192,K=28672",
        "value": dbytes / (dwall / args.steps) / 1e9,
        "unit": "GB/s",
        "ms_per_step": dwall / args.steps * 1e3,
        "roofline": {
            "kernel": dkernel,
            "bound": "hbm",
            "achieved": d_achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": d_achieved / HBM_PEAK_GBS,
            "traffic": dtraffic,
            "traffic_what": dtraffic_what,
            "launch_ms_mean": dev_ms,
            "algorithmic_bytes_per_launch": dbytes,
            "stream_ceiling_gbs": stream_p["stream_ceiling_gbs"],
            "frac_of_stream_ceiling": d_achieved / stream_p["stream_ceiling_gbs"],
            "stream_probe": stream_p,
        },
        "tile_major_weights": dtile,
        "batched_m32": dm32,
        "batched_m64": dbatched,
        "batched_m256": dmid,
        "prefill_m512": dprefill,
    }

    line = {
        "metric": "MXFP6 GEMM TFLOPS @8192^3 (% of MFMA peak); GB/s @M=16 decode",
        "value": value,
        "unit": "TFLOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": value / PUBLISHED_FP6_8192,
        "vs_baseline_note": "value (whole step from row-major inputs, back-to-back launches) / 2861.52, the reference's published FP6 GEMM at 8192^3 on MI355X; roofline.ref_protocol holds the per-launch figures under the reference's own protocol (fresh inputs, sync, one event pair per launch)",
        "value_prepared_weights": flops / (pwall / args.steps) / 1e12,
        "value_prepared_weights_note": "the same step with B and its scales converted to the tile-major weight format once, outside the timed region (mxfp6_blob_pack / mxfp6_tile_operand at load time): the pre-pass copies A only",
        "ms_per_step_prepared_weights": pwall / args.steps * 1e3,
        "dtype": "mxfp6 e2m3 x e2m3 (E8M0 block scales), f32 accumulate, bf16 out",
        "data": "synthetic",
        "config": {
            "workload": "BASELINE configs[1]: square MXFP6 e2m3 GEMM C=A.B^T, M=N=K=8192, N(0,1) sources quantised per 32-block, bf16 output",
            "M": M, "N": N, "K": K, "fmt_a": "e2m3", "fmt_b": "e2m3", "input_sets": 3,
            "inputs": "fp32 sources drawn on the CPU (numpy default_rng, seeds 1001 / 1002; sets 2 and 3 are the same sources with rows rotated), quantised by the library's GPU quantiser",
            "prewarm": f"{PREWARM_MS:.0f} ms of the same launches, untimed, in front of the warm-up steps of the 8192^3 loops (the power management's transient after idle)",
        },
        "pct_of_mfma_peak": 100.0 * value / MFMA_PEAK_TFLOPS,
        "roofline": roofline,
        "tile_major": tile_major,
        "cpu_baseline": cpu,
        "configs": configs,
        "decode": decode,
        "quantize": quant,
        "squares": squares,
        "device": torch.cuda.get_device_name(0),
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
