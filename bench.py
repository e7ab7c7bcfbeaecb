#!/usr/bin/env python3
"""Roofline bench of the decode GEMV path on one MI355X.

Workload (BASELINE config 2, the q4 batch-1 leg the headline metric is quoted on): one step =
one q4_0 decode GEMV (activation int8 preparation + GEMV kernel) over each of the four shapes
NxK = 4096x4096, 14336x4096, 4096x14336, 262144x2048, weights ~N(0,0.02) quantized by the aion
q4 quantizer, activations ~N(0,1), all resident in HBM before the timed region. Two full weight
sets alternate between steps (754 MB footprint) so that no step re-reads a weight that could
still sit in the 256 MB memory-side cache.

value   = algorithmic bytes of the step (N*K/32*18 + 4*(K+N) per shape) / step time, GB/s.
roofline = the same for the GEMV kernel alone, from per-launch stream events recorded inside the
timed region, against the 8 TB/s HBM peak.
cpu_baseline = the oracle's restatement of the aion CPU kernel for this op (packed int8 GEMM at
M=1, aion cpu/exec/matmul.zig) timed on this host's cores on a bounded sample.

`--sweep` adds the q8 legs and batch 4 / 8 (per-shape kernel GB/s) in a "sweep" object.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

SHAPES = [(4096, 4096), (14336, 4096), (4096, 14336), (262144, 2048)]   # N x K
HBM_PEAK_GBPS = 8000.0


def algorithmic_bytes(dtype_bytes, n, k, batch):
    return n * k // 32 * dtype_bytes + batch * (k + n) * 4


def synth_blocks(be, dtype, layout, n, k, seed):
    """Weights ~N(0,0.02) through the host quantizer. A 2^22-sample normal pool is tiled to the
    full size (timing does not depend on the values; the distribution per block is unchanged)."""
    rng = np.random.default_rng(seed)
    pool = (rng.standard_normal(1 << 22) * 0.02).astype(np.float32)
    total = n * k
    shape = (n, k) if layout == be.ROWS_NK else (k, n)
    reps = -(-total // pool.size)
    w = np.tile(pool, reps)[:total].reshape(shape)
    return be.quantize_blocks(dtype, w, 1 if layout == be.ROWS_NK else 0)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--sweep", action="store_true", help="also time q8 and batch 4/8 per shape")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this backend is single-GPU (aion runs one program on one device); --gpus %d is not supported" % args.gpus)

    from aion_amd import backend as be

    gpu = be.HipBackend(0)
    info = gpu.device_info()
    batch = 1
    n_sets = 2
    t0 = time.time()
    host_blocks = {}
    sets = []
    for s in range(n_sets):
        ws = []
        for (n, k) in SHAPES:
            if s == 0:
                host_blocks[(n, k)] = synth_blocks(be, be.Q4_0, be.KMAJOR_KN, n, k, seed=n * 31 + k)
            ws.append(gpu.upload_weight(be.Q4_0, be.KMAJOR_KN, n, k, host_blocks[(n, k)]))
        sets.append(ws)
    rng = np.random.default_rng(7)
    xs = [gpu.upload(rng.standard_normal((batch, k)).astype(np.float32)) for (_, k) in SHAPES]
    ys = [gpu.alloc(batch * n * 4) for (n, _) in SHAPES]
    setup_s = time.time() - t0

    def step(i):
        ws = sets[i % n_sets]
        for j in range(len(SHAPES)):
            gpu.step_matmul(ws[j], xs[j], batch, ys[j])

    for i in range(args.warmup):
        step(i)
    gpu.sync()
    ev0, ev1 = gpu.event(), gpu.event()
    gpu.profile_start()
    gpu.record(ev0)
    t_wall = time.perf_counter()
    for i in range(args.steps):
        step(args.warmup + i)
    gpu.record(ev1)
    gpu.sync()
    wall_ms = (time.perf_counter() - t_wall) * 1e3
    total_ms = gpu.elapsed_ms(ev0, ev1)
    prof = gpu.profile_stop()

    step_bytes = sum(algorithmic_bytes(18, n, k, batch) for (n, k) in SHAPES)
    ms_per_step = total_ms / args.steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    gemv = [ms for (name, ms) in prof if name == "gemv_q4"]
    assert len(gemv) == args.steps * len(SHAPES), (len(gemv), args.steps)
    avg_launch_ms = sum(gemv) / len(gemv)
    bytes_per_launch = step_bytes / len(SHAPES)
    achieved = bytes_per_launch / (avg_launch_ms * 1e-3) / 1e9
    per_shape = {}
    for j, (n, k) in enumerate(SHAPES):
        ms = sum(gemv[j::len(SHAPES)]) / args.steps
        per_shape["%dx%d" % (n, k)] = {"kernel_us": round(ms * 1e3, 2),
                                        "GBps": round(algorithmic_bytes(18, n, k, batch) / (ms * 1e-3) / 1e9, 1)}

    out = {
        "metric": "q4_gemv_hbm_GBps", "value": round(value, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8 dot, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": "config 2, q4_0 decode GEMV batch 1 over 4096x4096, 14336x4096, 4096x14336, 262144x2048 (one step = the four GEMVs incl. activation int8 preparation)",
                   "device": info["arch"], "cu_count": info["cu_count"], "weight_sets_rotated": n_sets,
                   "step_algorithmic_bytes": step_bytes, "wall_ms_per_step": round(wall_ms / args.steps, 5)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel": "gemv_q4", "avg_launch_us": round(avg_launch_ms * 1e3, 3),
                     "algorithmic_bytes_per_launch": bytes_per_launch, "per_shape": per_shape},
    }

    if args.sweep:
        out["sweep"] = run_sweep(gpu, be, host_blocks)

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(host_blocks, batch)

    out["config"]["setup_s"] = round(setup_s, 1)
    print(json.dumps(out))
    gpu.close()


def time_kernel(gpu, ws, x, y, m, name, iters=20):
    for i in range(3):
        gpu.step_matmul(ws[i % len(ws)], x, m, y)
    gpu.sync()
    gpu.profile_start()
    for i in range(iters):
        gpu.step_matmul(ws[i % len(ws)], x, m, y)
    prof = [ms for (nm, ms) in gpu.profile_stop() if nm == name]
    return sum(prof) / len(prof)


def run_sweep(gpu, be, q4_blocks):
    res = {}
    rng = np.random.default_rng(11)
    for dtype, layout, bb, kname in ((be.Q4_0, be.KMAJOR_KN, 18, "gemv_q4"), (be.Q8_0, be.ROWS_NK, 34, "gemv_q8")):
        for (n, k) in SHAPES:
            blocks = q4_blocks[(n, k)] if dtype == be.Q4_0 else synth_blocks(be, dtype, layout, n, k, seed=n + k)
            copies = max(2, min(64, int(600e6 // blocks.nbytes) + 1))   # > 2x the 256 MB memory-side cache
            ws = [gpu.upload_weight(dtype, layout, n, k, blocks) for _ in range(copies)]
            for m in (1, 4, 8):
                x = gpu.upload(rng.standard_normal((m, k)).astype(np.float32))
                y = gpu.alloc(m * n * 4)
                ms = time_kernel(gpu, ws, x, y, m, kname)
                by = algorithmic_bytes(bb, n, k, m)
                res["%s %dx%d b%d" % ("q4" if dtype == be.Q4_0 else "q8", n, k, m)] = {
                    "kernel_us": round(ms * 1e3, 2), "GBps": round(by / (ms * 1e-3) / 1e9, 1),
                    "frac_hbm_peak": round(by / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 3)}
                x.free(); y.free()
            for w in ws:
                w.free()
    return res


def cpu_baseline(host_blocks, batch):
    """The oracle (a C++ restatement of aion's CPU kernel for q4: int8 activations, packed int8 GEMM
    with kc=256) over the same step, threaded over output columns on this host."""
    from oracle import oracle as orc
    threads = min(16, os.cpu_count() or 1)
    rng = np.random.default_rng(7)
    xs = {(n, k): rng.standard_normal((batch, k)).astype(np.float32) for (n, k) in SHAPES}
    total_bytes = 0
    t0 = time.perf_counter()
    reps = 0
    while True:
        for (n, k) in SHAPES:
            orc.matmul_q_packed(orc.Q4_0, xs[(n, k)], host_blocks[(n, k)], n, threads=threads)
            total_bytes += algorithmic_bytes(18, n, k, batch)
        reps += 1
        if time.perf_counter() - t0 > 10.0 or reps >= 400:
            break
    dt = time.perf_counter() - t0
    return {"value": round(total_bytes / dt / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": "%d repetitions of the same four-shape q4 batch-1 step (%.1f s), oracle/aion_oracle.cpp orc_matmul_q_packed, -O3 x86-64-v3" % (reps, dt)}


if __name__ == "__main__":
    main()
