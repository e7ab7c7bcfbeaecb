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

Before anything is timed, one output per shape is compared with the oracle ("parity_check").

The same JSON line carries the two other metrics BASELINE.json names, in a "secondary" object, each with a roofline block of
its own: "prefill_gemm" (config 3's largest shape, M = 2048, N = 14336, K = 4096, q4: the exact int8 path and the bf16 MFMA
path, TFLOP/s against the named MFMA peak, with the tolerance class of each) and "decode" (config 5: the 26-layer decoder,
128-token prompt, greedy decode of 128 tokens at batch 1: tokens/s, ms/token, weight bytes streamed per second against the
HBM peak), plus "sweep": config 2's q8 legs and batch 4 / 8 per shape, and "attention": config 4's longest prompt and
largest decode shape. `--headline-only` skips the secondary object (and
with it every stream capture: the form to run under rocprofv3, which does not survive a capture in the traced process).
`--extras gemm,attention,decoder[,decoder_eager,session_decode,package,package_bench_shape,package_bench_shape_eager]` adds the full
config-3 and config-4 tables, the decoder with its CPU-oracle leg, the decoder as an unfused step list on the library's session
executor, and the package runner in an "extras" object.
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
CAL_ELEMS = 1 << 26   # the counter-calibration cast: 256 MiB read, 128 MiB written
# HBM bytes per launch (read + written) of the GEMV kernel of each shape, from FETCH_SIZE / WRITE_SIZE
# counter runs of this same command scaled by what the same counters read for the calibration cast
# (factors 1.9998 and 1.0000); the summary with the commands is profiles/gemv_q4_decode_bench_kernel_stats_and_traffic.md.
# Counters cannot be read from inside the process, so the figures are carried here.
MEASURED_TRAFFIC = {(4096, 4096): 9.656e6, (14336, 4096): 33.300e6, (4096, 14336): 33.886e6, (262144, 2048): 303.150e6}


SETTLE_MS = 80.0


def settle(gpu, fn, ms=SETTLE_MS):
    """Untimed load ahead of a measurement: `ms` milliseconds of the same calls, queued with no gap before what is timed.
    From idle the device needs 15-50 ms of a workload before its clocks settle (on one box: the four-GEMV step 70-73 us for
    the first 100 steps, 65.4 after 250; the bf16 GEMM 238-281 us for its first 20 launches, 220 after 100; prefill attention
    at L = 4096 105-112 us for its first 100 launches, 89 after 400), and what a decoder or a prompt sees is the settled rate. Returns the
    number of calls made."""
    ev0, ev1 = gpu.event(), gpu.event()
    gpu.record(ev0)
    for i in range(4):
        fn(i)
    gpu.record(ev1)
    gpu.sync()
    per = max(gpu.elapsed_ms(ev0, ev1) / 4, 1e-3)
    n = int(ms / per) + 1
    for i in range(n):
        fn(4 + i)
    return 4 + n


PROFILE_PAD = 4


def profiled(gpu, call, n):
    """The per-launch durations of n calls of call(i) (each launch carries its own start/stop events). PROFILE_PAD more calls
    are queued behind them and their entries dropped: the last launches before the host starts waiting for the stream now and
    then report durations of 300-600 us for a 5-50 us kernel (seen on fused and K-split GEMVs alike, always among the final
    four entries of a batch), which would move an average over few launches; the launches that count are never the last."""
    gpu.profile_start()
    for i in range(n + PROFILE_PAD):
        call(i)
    prof = gpu.profile_stop()
    per = len(prof) // (n + PROFILE_PAD)
    assert per * (n + PROFILE_PAD) == len(prof), "calls with a varying number of launches"
    return prof[:n * per]


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
    ap.add_argument("--sweep", action="store_true", help="(kept for compatibility: the sweep is part of the default run)")
    ap.add_argument("--headline-only", action="store_true", help="skip the secondary metrics (prefill GEMM, decode, sweep)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--extras", default="", help="comma list of sweep,gemm,attention,decoder,decode_stack,session_decode,package,package_bench_shape")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU (aion runs one program on one device, and no multi-GPU figure is asked for); "
                 "--gpus %d is not supported" % args.gpus)

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

    parity = check_against_oracle(gpu, be, sets, host_blocks, batch)

    def step(i):
        ws = sets[i % n_sets]
        for j in range(len(SHAPES)):
            gpu.step_matmul(ws[j], xs[j], batch, ys[j])

    # what the step launches, by instance name and grid, so that the line can be matched to a kernel trace
    launched = {}
    for j, (n, k) in enumerate(SHAPES):
        gpu.step_matmul(sets[0][j], xs[j], batch, ys[j])
        launched["%dx%d" % (n, k)] = gpu.last_launch()
    # from idle: the W warm-up steps and K timed steps as asked, with nothing queued ahead of them (the device has been idle
    # for a second); reported beside the settled figure
    gpu.sync()
    time.sleep(1.0)
    for i in range(args.warmup):
        step(i)
    ev0, ev1 = gpu.event(), gpu.event()
    gpu.record(ev0)
    for i in range(args.steps):
        step(args.warmup + i)
    gpu.record(ev1)
    gpu.sync()
    idle_ms_per_step = gpu.elapsed_ms(ev0, ev1) / args.steps

    settled = settle(gpu, step)          # device conditioning, reported in config; then the W warm-up steps as asked
    for i in range(args.warmup):
        step(i)
    gpu.sync()
    # pass 1: exactly K steps between two stream events -> value (launch by launch: a single execution of the same steps as one
    # recorded program was measured too - 66-76 us per step from run to run against a steady 67-68 here - and not adopted)
    ev0, ev1 = gpu.event(), gpu.event()
    gpu.record(ev0)
    t_wall = time.perf_counter()
    for i in range(args.steps):
        step(args.warmup + i)
    gpu.record(ev1)
    gpu.sync()
    wall_ms = (time.perf_counter() - t_wall) * 1e3
    total_ms = gpu.elapsed_ms(ev0, ev1)
    # pass 2: the same K steps again, every dispatch carrying its own start/stop events -> roofline
    # (kept apart from pass 1 because timed dispatches cannot be queued back to back)
    prof = profiled(gpu, lambda i: step(args.warmup + i), args.steps)
    # counter calibration: a plain streaming kernel of known size (f32 -> f16 cast: 4 B read and
    # 2 B written per element) so that a FETCH_SIZE / WRITE_SIZE counter run of this same command
    # holds its own scale factor
    cal_n = CAL_ELEMS
    cal_src, cal_dst = gpu.alloc(cal_n * 4), gpu.alloc(cal_n * 2)
    for _ in range(3):
        gpu.step_cast_f32_f16(cal_dst, cal_src, cal_n)
    gpu.sync()
    cal_src.free(); cal_dst.free()

    # the device's practical read rate on the same byte counts: a plain streaming-read kernel over a region
    # of a 1 GiB buffer that moves with every launch (nothing is re-read before 1 GiB of other data went by)
    read_us = {}
    rd_buf, rd_sink = gpu.alloc(1 << 30), gpu.alloc(16)
    rd_at = 0
    for (n, k) in SHAPES:
        nb = algorithmic_bytes(18, n, k, batch) // 16 * 16
        gpu.probe_stream_read(rd_buf, 0, 1 << 30, rd_sink)         # first touch of the buffer / evict the previous shape
        gpu.sync()
        gpu.profile_start()
        for _ in range(20):
            if rd_at + nb > (1 << 30):
                rd_at = 0
            gpu.probe_stream_read(rd_buf, rd_at, nb, rd_sink)
            rd_at += nb
        tms = sorted(ms for (nm, ms) in gpu.profile_stop() if nm == "stream_read")
        read_us["%dx%d" % (n, k)] = tms[len(tms) // 2] * 1e3
    rd_buf.free(); rd_sink.free()

    step_bytes = sum(algorithmic_bytes(18, n, k, batch) for (n, k) in SHAPES)
    ms_per_step = total_ms / args.steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # every profile entry is one dispatch's own start/stop timestamps (what a kernel trace reports)
    gemv = [ms for (name, ms) in prof if name.startswith("gemv_q4")]
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
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "config 2, q4_0 decode GEMV batch 1 over 4096x4096, 14336x4096, 4096x14336, 262144x2048 (one step = the four GEMVs incl. activation int8 preparation)",
                   "device": info["arch"], "cu_count": info["cu_count"], "weight_sets_rotated": n_sets,
                   "step_algorithmic_bytes": step_bytes, "wall_ms_per_step": round(wall_ms / args.steps, 5),
                   "from_idle": {"ms_per_step": round(idle_ms_per_step, 5),
                                 "GBps": round(sum(algorithmic_bytes(18, n, k, batch) for (n, k) in SHAPES) / (idle_ms_per_step * 1e-3) / 1e9, 1),
                                 "frac_of_peak": round(sum(algorithmic_bytes(18, n, k, batch) for (n, k) in SHAPES) / (idle_ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                                 "note": "the same W warm-up and K timed steps after one idle second, nothing queued ahead of them (stream events around the K steps)"},
                   "settling": "%d untimed steps (%.0f ms) ahead of the warm-up steps, and the same %.0f ms of load ahead of every "
                               "secondary figure: the first 15-50 ms of a workload after idle run 5-25 %% slower while the clocks settle"
                               % (settled, SETTLE_MS, SETTLE_MS)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": round(sum(MEASURED_TRAFFIC[sh] for sh in SHAPES) / len(SHAPES)),
                     "kernel": "gemv_q4 (gemv_fused_kernel for K <= 4096, gemv_ksplit_kernel above; activation preparation inside both)",
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, profiles/gemv_q4_decode_bench_kernel_stats_and_traffic.md", "avg_launch_us": round(avg_launch_ms * 1e3, 3),
                     "algorithmic_bytes_per_launch": bytes_per_launch, "per_shape": per_shape, "launched": launched,
                     "traffic_per_shape": {"%dx%d" % sh: MEASURED_TRAFFIC[sh] for sh in SHAPES},
                     "plain_read_same_bytes": {
                         "kernel_us": {sh: round(us, 2) for sh, us in read_us.items()},
                         "GBps": round(step_bytes / (sum(read_us.values()) * 1e-6) / 1e9, 1),
                         "gemv_rate_over_plain_read_rate": round(sum(read_us.values()) / (avg_launch_ms * 1e3 * len(SHAPES)), 3),
                         "note": "stream_read_kernel: reads only (one contiguous 4 KiB piece per wavefront, 16-byte non-temporal loads), cold data, same byte count per launch"}},
    }

    out["config"]["arithmetic"] = "int8 activations x int4 weights, exact i32 block dots (v_dot4_i32_i8), f32 scale-accumulate"
    out["parity_check"] = parity

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(host_blocks, batch)

    extras = [e for e in args.extras.split(",") if e]
    for ws in sets:
        for w in ws:
            w.free()
    for t in xs + ys:
        t.free()
    if not args.headline_only:
        out["secondary"] = {"prefill_gemm": run_gemm_headline(gpu, be), "decode": run_decode_headline(gpu, be),
                            "sweep": run_sweep(gpu, be, host_blocks), "attention": run_attention_headline(gpu, be)}
    if extras:
        out["extras"] = {}
        if "sweep" in extras:          # the sweep of the default run on its own (for a kernel trace: --headline-only --extras sweep)
            out["extras"]["sweep"] = run_sweep(gpu, be, host_blocks)
        if "gemm" in extras:
            out["extras"]["prefill_gemm"] = run_gemm(gpu, be)
        if "attention" in extras:
            out["extras"]["attention"] = run_attention(gpu, be)
        if "decoder" in extras:
            out["extras"]["decoder"] = run_decoder(gpu, be, with_cpu=not args.no_cpu)
        if "decode_stack" in extras or "decode_stack_only" in extras:
            out["extras"]["decode_stack"] = run_decode_stack(gpu, be, compare="decode_stack" in extras)
        if "session_decode" in extras:
            out["extras"]["session_decode"] = run_session_decode(gpu, be)
        if "decoder_eager" in extras:
            out["extras"]["decoder_eager"] = run_decoder_eager(gpu, be)
        if "package" in extras:
            out["extras"]["package"] = run_package(gpu, be)
        if "package_bench_shape" in extras:
            out["extras"]["package_bench_shape"] = run_package_bench_shape(gpu, be)
        if "package_bench_shape_eager" in extras:
            out["extras"]["package_bench_shape_eager"] = run_package_bench_shape(gpu, be, eager=True)

    out["config"]["setup_s"] = round(setup_s, 1)
    print(json.dumps(out))
    gpu.close()


def check_against_oracle(gpu, be, sets, host_blocks, batch):
    """One output per shape and weight set against the oracle (the checker, never the thing measured): the bar of the GPU
    parity tests, max|err| <= 1e-5 * rms(ref). Raises if a shape fails."""
    from oracle import oracle as orc
    rng = np.random.default_rng(123)
    worst = {}
    for j, (n, k) in enumerate(SHAPES):
        x_h = rng.standard_normal((batch, k)).astype(np.float32)
        want = orc.matmul_q_packed(orc.Q4_0, x_h, host_blocks[(n, k)], n, threads=min(16, os.cpu_count() or 1))
        rms = float(np.sqrt((want.astype(np.float64) ** 2).mean()))
        x, y = gpu.upload(x_h), gpu.alloc(batch * n * 4)
        for ws in sets:
            gpu.step_matmul(ws[j], x, batch, y)
            err = float(np.abs(gpu.download(y, np.float32, (batch, n)) - want).max()) / rms
            worst["%dx%d" % (n, k)] = max(worst.get("%dx%d" % (n, k), 0.0), err)
        x.free(); y.free()
    bad = {sh: e for sh, e in worst.items() if not e < 1e-5}
    if bad:
        raise SystemExit("bench.py: GEMV output differs from the oracle: %r" % bad)
    return {"against": "oracle matmul_q_packed (aion's CPU algorithm for q4)", "bar": "max|err| <= 1e-5 * rms(ref)",
            "max_err_over_rms": {sh: float("%.3g" % e) for sh, e in worst.items()}}


def run_gemm_headline(gpu, be):
    """BASELINE config 3's largest shape, q4: M = 2048 tokens, K = 4096, N = 14336. Both prefill paths, kernel time from
    per-launch events (a call may be more than one launch)."""
    rng = np.random.default_rng(3)
    m, n, k = 2048, 14336, 4096
    w = gpu.upload_weight(be.Q4_0, be.KMAJOR_KN, n, k, synth_blocks(be, be.Q4_0, be.KMAJOR_KN, n, k, seed=n))
    x = gpu.upload(rng.standard_normal((m, k)).astype(np.float32))
    y = gpu.alloc(m * n * 4)
    res = {"workload": "config 3: q4_0 weight 14336x4096, M = 2048 tokens, f32 activations N(0,1), f32 output", "flop": 2.0 * m * n * k}
    for mode, kname, peak, key, note in (
            (be.GEMM_BF16_MFMA_ALWAYS, "gemm_bf16", "bf16", "bf16_mfma",
             "weights read from the bf16 copy the context keeps of them (built at the first bf16 GEMM of a weight), activations rounded to bf16 by a launch of their own, f32 accumulate: tolerance class 1e-2 (tests: <= 1e-2 * rms vs the "
             "f32-activation oracle, NMSE <= 1e-4 vs aion's int8-activation CPU path)"),
            (be.GEMM_EXACT_I8, "gemm_i8_q4", "int8", "exact_i8",
             "aion's arithmetic (int8 activations per 32-block, exact i32 block dots, f32 scale-accumulate): tolerance class 2e-3, "
             "observed 1e-6. The parity path, not the throughput path: both operands carry a scale per 32-block, so every 16x16x32 "
             "MFMA is followed by 12 VALU instructions of rescaling, which bounds it near 15 % of the int8 peak")):
        gpu.set_gemm_mode(mode)
        gpu.step_matmul(w, x, m, y)
        settle(gpu, lambda i: gpu.step_matmul(w, x, m, y))
        prof = profiled(gpu, lambda i: gpu.step_matmul(w, x, m, y), 20)
        # every launch of a call counts: the activation's bf16 rounding / int8 preparation runs as a launch of its own
        per_name = {}
        for nm, t in prof:
            per_name.setdefault(nm, []).append(t)
        assert kname in per_name, (kname, sorted(per_name))
        ms = sum(t for _, t in prof) / 20
        main_ms = sum(per_name[kname]) / 20
        tf = 2.0 * m * n * k / (ms * 1e-3) / 1e12
        res[key] = {"call_ms": round(ms, 4), "launches_per_call": len(prof) // 20,
                    "launches": {nm: round(sum(v) / 20, 4) for nm, v in per_name.items()},
                    "TFLOPs": round(tf, 1), "TFLOPs_main_kernel_alone": round(2.0 * m * n * k / (main_ms * 1e-3) / 1e12, 1), "note": note,
                    "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": MFMA_PEAK[peak], "unit": "TFLOP/s",
                                 "frac": round(tf / MFMA_PEAK[peak], 4), "traffic": None, "peak_named": "dense " + peak + " MFMA",
                                 "counts": "every launch of the call (the sum of their durations)"}}
    # the bf16 kernel's second weight form: no bf16 copy, the quant blocks are converted while they are staged (same bits out)
    gpu.set_gemm_mode(be.GEMM_BF16_MFMA_ALWAYS)
    gpu.set_bf16_weight_copies(False)
    w.drop_bf16()
    gpu.step_matmul(w, x, m, y)
    settle(gpu, lambda i: gpu.step_matmul(w, x, m, y))
    prof = profiled(gpu, lambda i: gpu.step_matmul(w, x, m, y), 20)
    ms = sum(t for _, t in prof) / 20
    res["bf16_mfma_blocks_converted_while_staged"] = {
        "call_ms": round(ms, 4), "launches_per_call": len(prof) // 20, "TFLOPs": round(2.0 * m * n * k / (ms * 1e-3) / 1e12, 1),
        "bf16_copy_bytes": int(gpu.bf16_copy_stats()[1]),
        "note": "aionhip_set_bf16_weight_copies(ctx, 0): nothing resident beyond the q4 weight; slower than the copy form, which stays the default"}
    gpu.set_bf16_weight_copies(True)
    gpu.set_gemm_mode(be.GEMM_EXACT_I8)
    x.free(); y.free(); w.free()
    return res


def run_decode_headline(gpu, be):
    """BASELINE config 5: the synthetic 26-layer decoder, 128-token prompt, greedy decode of 128 tokens at batch 1 (program
    replay; the tokens are logged on the device and read back once, and the loop with a read-back per step is timed beside it). The arithmetic is checked per node at full size in tests/test_gpu_config5.py."""
    from aion_amd.decoder import Decoder, DecoderConfig, SyntheticWeights, weight_shapes
    cfg = DecoderConfig()
    t0 = time.time()
    dec = Decoder(gpu, cfg, SyntheticWeights(cfg, 0))
    setup_s = time.time() - t0
    prompt = np.random.default_rng(5).integers(0, cfg.vocab, 128).astype(np.int32)
    weight_bytes = sum(n * k // 32 * 18 for (n, k) in weight_shapes(cfg).values())
    dec.prefill(prompt); dec.reset()             # warm-up: scratch reaches its final size
    gpu.sync()
    t = time.perf_counter()
    first = dec.prefill(prompt)
    prefill_ms = (time.perf_counter() - t) * 1e3
    # what is checked here: the first decode step issued launch by launch and the first replay of the recorded program give the
    # same logits, bit for bit (the program is the same launches); below, the two 128-token loops give the same tokens
    tok_eager = dec.decode_step_eager(first)
    logits_eager = dec.logits_host()
    dec.reset()
    assert dec.prefill(prompt) == first
    dec.begin_decode(first)
    gpu.sync()
    tok_replay = dec.decode_step()
    logits_equal = bool(np.array_equal(dec.logits_host(), logits_eager)) and tok_replay == tok_eager
    if not logits_equal:
        raise SystemExit("bench.py: the replayed decode program and the eager launches disagree on the first step's logits")
    dec.reset()
    assert dec.prefill(prompt) == first
    dec.begin_decode(first)
    gpu.sync()
    # Two generations of 128 tokens from the same prompt. The first reads every token back (4 bytes, a synchronisation per
    # step); it also is the load under which the device settles. The second is 128 replays of the decode program back to
    # back: the loop state and the produced tokens stay on the device and the tokens are read back once at the end.
    t = time.perf_counter()
    toks_each = [dec.decode_step() for _ in range(128)]
    gpu.sync()
    decode_each_s = time.perf_counter() - t
    dec.reset()
    first2 = dec.prefill(prompt)
    dec.begin_decode(first2)
    gpu.sync()
    t = time.perf_counter()
    toks = dec.decode_run(128)
    gpu.sync()
    decode_s = time.perf_counter() - t
    assert first2 == first and list(toks) == toks_each, "the two decode loops disagree"
    tok_s = 128 / decode_s
    gbps = weight_bytes / (decode_s / 128) / 1e9
    res = {"workload": "config 5: 26 layers, hidden 2048, 8 q / 1 kv heads x 256, GeGLU 8192, vocab 262144, q4_0 weights, f16 KV cache, "
                       "prompt 128, greedy 128, batch 1",
           "decode_tokens_per_s": round(tok_s, 1), "decode_ms_per_token": round(decode_s / 128 * 1e3, 4),
           "decode_tokens_per_s_read_back_every_step": round(128 / decode_each_s, 1),
           "prefill_128_ms": round(prefill_ms, 3), "prefill_tokens_per_s": round(128 / (prefill_ms * 1e-3), 1),
           "checked": {"here": "first decode step: logits of the replayed program == logits of the same step issued launch by launch (bit-equal, "
                               "262144 values) and the same token; the 128 tokens of the read-back-per-step loop == the 128 of the replay loop",
                       "not_here": "agreement with aion's arithmetic: per node at this full size against the oracle in tests/test_gpu_config5.py "
                                   "(embedding, every block's q/k/v, attention, o, gate/up, down at their parity bars) and end to end on the small "
                                   "decoder in tests/test_gpu_decoder.py; end-to-end logits at 26 layers are not a parity criterion (int8 "
                                   "re-quantisation of activations makes two correct schedules drift 0.1-0.2 rms apart)"},
           "weight_bytes_per_token": weight_bytes, "program_nodes": int(gpu.program_node_count(dec.program)), "setup_s": round(setup_s, 1),
           "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(gbps / HBM_PEAK_GBPS, 4),
                        "traffic": None, "note": "algorithmic bytes = every q4_0 weight read once per token (KV cache and activations are < 1 % at this "
                                                 "length); a decode step is a chain of ~140 dependent launches, so latency per launch, not bandwidth, bounds it"}}
    dec.close()
    return res


def time_kernel(gpu, ws, x, y, m, name, iters=20):
    settle(gpu, lambda i: gpu.step_matmul(ws[i % len(ws)], x, m, y), 20.0)     # the sweep's launches follow each other: a short load each
    prof = profiled(gpu, lambda i: gpu.step_matmul(ws[i % len(ws)], x, m, y), iters)
    names = (name,) if isinstance(name, str) else tuple(name)
    assert any(nm.startswith(names) for nm, _ms in prof), (name, prof[:4])
    per = len(prof) // iters                      # every launch of the call: the activation preparation and the GEMV(s)
    calls = sorted(sum(ms for _nm, ms in prof[i * per:(i + 1) * per]) for i in range(iters))
    return calls[iters // 2]


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
                # five to eight rows over a K past 4096 run on the exact GEMM's 16-row tile, everything else on a GEMV kernel
                ms = time_kernel(gpu, ws, x, y, m, (kname, "gemm_i8_" + kname[-2:]) if m >= 5 and k > 4096 else kname)
                by = algorithmic_bytes(bb, n, k, m)
                ll = gpu.last_launch()
                res["%s %dx%d b%d" % ("q4" if dtype == be.Q4_0 else "q8", n, k, m)] = {
                    "kernels": gpu.last_kernel(), "launched": "%s grid %s x %d" % (ll["kernel"].replace("(anonymous namespace)::", ""), ll["grid"], ll["block"][0]),
                    "kernel_us": round(ms * 1e3, 2), "GBps": round(by / (ms * 1e-3) / 1e9, 1),
                    "frac_hbm_peak": round(by / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 3)}
                x.free(); y.free()
            for w in ws:
                w.free()
    return res


MFMA_PEAK = {"bf16": 2500.0, "int8": 5000.0}   # dense TFLOP/s (TOP/s)


def run_gemm(gpu, be):
    """BASELINE config 3: M in {512, 2048}, K = 4096, N in {4096, 14336}; kernel time from per-launch events."""
    res = {}
    rng = np.random.default_rng(3)
    k = 4096
    for dtype, layout, tag in ((be.Q4_0, be.KMAJOR_KN, "q4"), (be.Q8_0, be.ROWS_NK, "q8")):
        for n in (4096, 14336):
            w = gpu.upload_weight(dtype, layout, n, k, synth_blocks(be, dtype, layout, n, k, seed=n))
            for m in (512, 2048):
                x = gpu.upload(rng.standard_normal((m, k)).astype(np.float32))
                y = gpu.alloc(m * n * 4)
                for mode, kname, peak in ((be.GEMM_BF16_MFMA_ALWAYS, "gemm_bf16", "bf16"), (be.GEMM_EXACT_I8, "gemm_i8_" + tag, "int8")):
                    gpu.set_gemm_mode(mode)
                    gpu.step_matmul(w, x, m, y)
                    settle(gpu, lambda i: gpu.step_matmul(w, x, m, y), 40.0)
                    gpu.profile_start()
                    t0 = time.perf_counter()
                    for _ in range(10):
                        gpu.step_matmul(w, x, m, y)
                    prof = [ms for (nm, ms) in gpu.profile_stop() if nm == kname]
                    wall = (time.perf_counter() - t0) / 10
                    ms = sum(prof) / 10             # a call may be more than one launch of this kernel
                    tf = 2.0 * m * n * k / (ms * 1e-3) / 1e12
                    res["%s M%d N%d %s" % (tag, m, n, "bf16" if mode == be.GEMM_BF16_MFMA_ALWAYS else "exact_i8")] = {
                        "kernel_ms": round(ms, 4), "step_wall_ms": round(wall * 1e3, 4), "TFLOPs": round(tf, 1),
                        "frac_mfma_peak": round(tf / MFMA_PEAK[peak], 4), "peak": peak}
                x.free(); y.free()
            w.free()
    gpu.set_gemm_mode(be.GEMM_EXACT_I8)
    return res


def _bf16_bits(x):
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def run_attention(gpu, be, prefill=(1024, 2048, 4096), decode=((1024, 1), (1024, 8), (4096, 1), (4096, 8), (16384, 1), (16384, 8))):
    """BASELINE config 4: 8 q heads / 1 kv head, head_dim 256, bf16 Q/K/V, scale 1/16, causal."""
    res = {}
    rng = np.random.default_rng(4)
    Hq, Hkv, D = 8, 1, 256

    def timed(name, shape, bufs, pos=None, kl=None, iters=10):
        settle(gpu, lambda i: gpu.step_attention(bufs[3], bufs[0], bufs[1], bufs[2], shape, 1 / 16.0, q_dtype=be.BF16, kv_dtype=be.BF16,
                                                 query_positions=pos, kv_lengths=kl))
        gpu.profile_start()
        for _ in range(iters):
            gpu.step_attention(bufs[3], bufs[0], bufs[1], bufs[2], shape, 1 / 16.0, q_dtype=be.BF16, kv_dtype=be.BF16,
                               query_positions=pos, kv_lengths=kl)
        prof = gpu.profile_stop()
        # per call: the sum of its kernels (split + merge); median over calls (the first call of a kernel
        # shape may still carry one-time set-up)
        kernels = [ms for (nm, ms) in prof if nm in name]
        per = len(kernels) // iters
        per_call = sorted(sum(kernels[i * per:(i + 1) * per]) for i in range(iters))
        return per_call[iters // 2]

    for L in prefill:
        q = gpu.upload(_bf16_bits(rng.standard_normal((1, L, Hq, D))))
        k = gpu.upload(_bf16_bits(rng.standard_normal((1, L, Hkv, D))))
        v = gpu.upload(_bf16_bits(rng.standard_normal((1, L, Hkv, D))))
        o = gpu.alloc(L * Hq * D * 4)
        # the 128-row prefill kernel; where its row tiles alone would leave CUs idle (L = 1024, 2048) every row
        # tile's key range is cut into segments and a merge pass folds them (both kernels are timed)
        ms = timed(("attn_prefill", "attn_flash_split", "attn_merge"), (1, L, L, Hq, Hkv, D, D), (q, k, v, o))
        flops = 4.0 * Hq * D * L * (L + 1) / 2
        tf = flops / (ms * 1e-3) / 1e12
        res["prefill L%d" % L] = {"kernel_ms": round(ms, 4), "TFLOPs": round(tf, 1), "frac_mfma_peak": round(tf / MFMA_PEAK["bf16"], 4),
                                  "kernel": gpu.last_kernel()}
        for t in (q, k, v, o):
            t.free()
    for T, B in decode:
        if True:
            q = gpu.upload(_bf16_bits(rng.standard_normal((B, 1, Hq, D))))
            k = gpu.upload(_bf16_bits(rng.standard_normal((B, T, Hkv, D))))
            v = gpu.upload(_bf16_bits(rng.standard_normal((B, T, Hkv, D))))
            o = gpu.alloc(B * Hq * D * 4)
            pos = gpu.upload(np.full((B, 1), T - 1, np.int32))
            kl = gpu.upload(np.full((B,), T, np.int32))
            ms = timed(("attn_flash_split", "attn_merge"), (B, 1, T, Hq, Hkv, D, D), (q, k, v, o), pos, kl, iters=20)
            by = B * 2 * T * Hkv * D * 2 + B * Hq * D * (2 + 4)
            res["decode T%d B%d" % (T, B)] = {"kernel_us": round(ms * 1e3, 2), "GBps": round(by / (ms * 1e-3) / 1e9, 1),
                                              "frac_hbm_peak": round(by / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
            for t in (q, k, v, o, pos, kl):
                t.free()
    return res


def run_attention_headline(gpu, be):
    """Config 4 in the default line: the longest prompt and the largest decode shape of the table `--extras attention`
    prints in full, each with its roofline block."""
    full = run_attention(gpu, be, prefill=(4096,), decode=((16384, 8),))
    pf, dc = full["prefill L4096"], full["decode T16384 B8"]
    return {
        "workload": "config 4: 8 q heads / 1 kv head, head size 256, bf16 Q/K/V, scale 1/16, causal",
        "prefill_L4096": {"kernel_ms": pf["kernel_ms"], "TFLOPs": pf["TFLOPs"],
                          "note": "tile kernel + merge of its two key segments; flop = 4 Hq D L (L + 1) / 2",
                          "roofline": {"bound": "mfma", "achieved": pf["TFLOPs"], "peak": MFMA_PEAK["bf16"], "unit": "TFLOP/s",
                                       "frac": pf["frac_mfma_peak"], "traffic": None, "peak_named": "dense bf16 MFMA"}},
        "decode_T16384_B8": {"kernel_us": dc["kernel_us"],
                             "note": "split-K kernel + merge; bytes = K and V of the cache once, queries and outputs",
                             "roofline": {"bound": "hbm", "achieved": dc["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                                          "frac": dc["frac_hbm_peak"], "traffic": None}},
    }


def run_decoder_eager(gpu, be, steps=8):
    """The config-5 decode step issued launch by launch (no program replay): the form a kernel trace can
    attribute per kernel (rocprofv3 does not survive stream capture in the traced process)."""
    from aion_amd.decoder import Decoder, DecoderConfig, SyntheticWeights
    cfg = DecoderConfig()
    dec = Decoder(gpu, cfg, SyntheticWeights(cfg, 0))
    prompt = np.random.default_rng(5).integers(0, cfg.vocab, 128).astype(np.int32)
    tok = dec.prefill(prompt)
    gpu.sync()
    t = time.perf_counter()
    for _ in range(steps):
        tok = dec.decode_step_eager(tok)
    gpu.sync()
    return {"steps": steps, "eager_ms_per_token": round((time.perf_counter() - t) / steps * 1e3, 4)}


def run_session_decode(gpu, be):
    """Config 5 as a compiled program reaches a backend: one record per graph step (19 per block, nothing pre-fused), run by the
    library's session executor (aionhip_session_execute), recorded as a program and replayed; beside the hand-routed Decoder
    over the same weights, whose prefill logits and 128 tokens it must reproduce."""
    from aion_amd.decoder import Decoder, DecoderConfig, SessionDecoder, SyntheticWeights
    cfg = DecoderConfig()
    w = SyntheticWeights(cfg, 0)
    prompt = np.random.default_rng(5).integers(0, cfg.vocab, 128).astype(np.int32)
    dec, ses = Decoder(gpu, cfg, w), SessionDecoder(gpu, cfg, w)
    ta, tb = dec.prefill(prompt), ses.prefill(prompt)
    prefill_equal = bool(np.array_equal(dec.logits_host(), ses.logits_host())) and ta == tb
    records = len(ses._program(1, advance=True)[1].records)
    dec.begin_decode(ta)
    ses.begin_decode(tb)
    want = [dec.decode_step() for _ in range(128)]
    got = [ses.decode_step() for _ in range(128)]
    res = {"step_records_per_token": records, "calls_per_token_after_folding": ses.calls_per_step,
           "program_nodes": int(gpu.program_node_count(ses.program)), "prefill_logits_equal": prefill_equal, "tokens_equal": got == want}
    for name, d in (("session", ses), ("hand_routed", dec)):
        d.pos = 0
        d.begin_decode(d.prefill(prompt))
        gpu.sync()
        t = time.perf_counter()
        for _ in range(128):
            d.decode_step(read_token=False)
        gpu.sync()
        dt = time.perf_counter() - t
        res[name] = {"decode_ms_per_token": round(dt / 128 * 1e3, 4), "decode_tokens_per_s": round(128 / dt, 1)}
    t = time.perf_counter()
    ses.pos = 0
    ses.prefill(prompt)
    gpu.sync()
    res["session"]["prefill_128_ms"] = round((time.perf_counter() - t) * 1e3, 3)
    dec.close(); ses.close()
    return res


def run_decode_stack(gpu, be, compare=True):
    """Config 5's decode step as ONE cooperative launch for all 26 blocks (aionhip_step_decoder_stack) beside the replayed
    program of the default path: ms per token of both, whether their 128 tokens agree, the launches of a step with their
    durations, and the kernel's own time stamps (100 MHz counter, relative to the start of a block's attention) for two blocks."""
    from aion_amd.decoder import Decoder, DecoderConfig, SyntheticWeights
    cfg = DecoderConfig()
    w = SyntheticWeights(cfg, 0)
    prompt = np.random.default_rng(5).integers(0, cfg.vocab, 128).astype(np.int32)
    res, toks = {}, {}
    for mode in ((True, False) if compare else (True,)):     # (a kernel trace cannot follow the recording of a program)
        dec = Decoder(gpu, cfg, w, one_launch=mode)
        dec.prefill(prompt); dec.reset(); gpu.sync()
        dec.begin_decode(dec.prefill(prompt)); gpu.sync()
        dec.decode_run(64); gpu.sync()                                  # settle
        dec.reset(); dec.begin_decode(dec.prefill(prompt)); gpu.sync()
        t = time.perf_counter()
        toks[mode] = list(dec.decode_run(128))
        gpu.sync()
        dt = time.perf_counter() - t
        key = "one_launch" if mode else "replayed_program"
        res[key] = {"decode_ms_per_token": round(dt / 128 * 1e3, 4), "decode_tokens_per_s": round(128 / dt, 1)}
        if mode:
            dec.reset(); dec.begin_decode(dec.prefill(prompt)); gpu.sync()
            gpu.profile_start()
            for _ in range(20):
                dec._step_on_device()
            agg = {}
            for nm, ms in gpu.profile_stop():
                agg.setdefault(nm, []).append(ms)
            res[key]["launches_us"] = {nm: round(1e3 * sum(v) / len(v), 2) for nm, v in agg.items()}
            st = gpu.zeros(2 * cfg.layers * 10 * 8)
            gpu.decoder_stack_set_stamps(dec.stack, st)
            dec._step_on_device(); gpu.sync()
            gpu.decoder_stack_set_stamps(dec.stack, None)
            v = gpu.download(st, np.int64, (2, cfg.layers, 10)).astype(np.float64) / 100.0      # microseconds
            names_a = ["attention_start", "attention_end", "q_arrived", "attention_out_published", "o_in", "o_out", "ffn_in", "ffn_out", "down_in", "down_out"]
            names_m = ["block_input_arrived", "qkv_published", "unused_2", "unused_3", "o_in", "o_out", "ffn_in", "ffn_out", "down_in", "down_out"]
            for l in (3, 12):
                t0 = v[0, l, 0]
                res[key]["block_%d_us_since_attention_start" % l] = {
                    "attention_workgroup": {nm: round(x - t0, 2) for nm, x in zip(names_a, v[0, l]) if x > 0},
                    "a_matmul_workgroup": {nm: round(x - t0, 2) for nm, x in zip(names_m, v[1, l]) if x > 0}}
            res[key]["block_period_us"] = [round(float(x), 2) for x in np.diff(v[0, :, 3])[:8]]
            st.free()
        dec.close()
    if compare:
        res["tokens_equal"] = toks[True] == toks[False]
    return res


def run_package(gpu, be):
    """BASELINE config 5 as a `.aion` package: written by oracle/aion_writer.py (the reference's writer cannot run
    here), read by aion_amd/aion_file.py, scheduled and run by aion_amd/package.py. Same weights as run_decoder."""
    from aion_amd import aion_file
    from aion_amd.decoder import DecoderConfig, SyntheticWeights
    from aion_amd.package import PackageRunner
    from oracle import aion_writer                       # test infrastructure: only used to make the input file
    cfg = DecoderConfig()
    t0 = time.time()
    weights = SyntheticWeights(cfg, 0)
    d = dict(layers=cfg.layers, hidden=cfg.hidden, heads=cfg.heads, kv_heads=cfg.kv_heads, head_dim=cfg.head_dim, ffn=cfg.ffn,
             vocab=cfg.vocab, eps=cfg.eps, rope_base=cfg.rope_base, wdtype="q4_0")
    data = aion_writer.build_decoder_package(d, weights.blocks, weights.embed())
    t_write = time.time() - t0
    t0 = time.time()
    pkg = aion_file.parse(data)
    t_parse = time.time() - t0
    run = PackageRunner(gpu, pkg, capacity=cfg.max_seq)
    prompt = np.random.default_rng(5).integers(0, cfg.vocab, 128).astype(np.int32)
    t0 = time.time()
    run.run(prompt); run.reset()                         # uploads the weights, builds the 128-token plan
    t_first = time.time() - t0
    gpu.sync()
    t = time.perf_counter()
    tok = int(run.run(prompt)["next_token"][0, -1])
    prefill_ms = (time.perf_counter() - t) * 1e3
    run.begin_decode(tok)
    gpu.sync()
    t = time.perf_counter()
    run.decode_run(127)                          # tokens logged on the device, read back once
    gpu.sync()
    decode_s = time.perf_counter() - t
    res = {"file_bytes": len(data), "nodes": len(pkg.nodes), "initializers": len(pkg.tensors),
           "write_s": round(t_write, 1), "parse_s": round(t_parse, 3), "upload_and_plan_s": round(t_first, 1),
           "steps_prefill_128": run.step_count(128), "steps_decode": run.step_count(1),
           "program_nodes": int(gpu.program_node_count(run.program)),
           "prefill_128_ms": round(prefill_ms, 3), "decode_tokens_per_s": round(127 / decode_s, 1),
           "decode_ms_per_token": round(decode_s / 127 * 1e3, 4)}
    run.close()
    return res


def run_package_bench_shape(gpu, be, eager=False):
    """eager: the single-token steps are issued launch by launch (no program replay), the form a kernel trace can
    attribute per kernel. A package with the block structure of aion's own bench model (src/bench/models.zig:433-536: tied row-quantized
    q8_0 table, scaled embedding, per-head q/k/v norms, norms on the block outputs, local layers on 512-row rings beside
    every fifth layer global, soft-capped logits) at BASELINE config 5's sizes, through the package runner. Random
    weights; the arithmetic is checked on a small instance of the same writer in the GPU tests."""
    from aion_amd import aion_file
    from aion_amd.decoder import DecoderConfig, SyntheticWeights
    from aion_amd.package import PackageRunner
    from oracle import aion_writer                       # test infrastructure: only used to make the input file
    cfg = DecoderConfig()
    weights = SyntheticWeights(cfg, 0)
    d = dict(layers=cfg.layers, hidden=cfg.hidden, heads=cfg.heads, kv_heads=cfg.kv_heads, head_dim=cfg.head_dim, ffn=cfg.ffn,
             vocab=cfg.vocab, eps=cfg.eps, rope_base_local=10000.0, rope_base_global=1000000.0, local_window=512, global_every=5,
             logit_softcap=30.0, wdtype="q4_0")
    rng = np.random.default_rng(11)
    gammas = {}
    for l in range(cfg.layers):
        for n, width in (("norm_in", cfg.hidden), ("q_norm", cfg.head_dim), ("k_norm", cfg.head_dim), ("v_norm", cfg.head_dim),
                         ("norm_attn", cfg.hidden), ("norm_ffn_in", cfg.hidden), ("norm_ffn", cfg.hidden)):
            gammas["l%d.%s" % (l, n)] = ((0.35 if n in ("q_norm", "k_norm") else 1.0) * (1 + 0.1 * rng.standard_normal(width))).astype(np.float32)
    gammas["norm_f"] = np.ones(cfg.hidden, np.float32)
    t0 = time.time()
    table = be.quantize_blocks(be.Q8_0, weights.embed(), 1)
    data = aion_writer.build_sandwich_decoder_package(d, weights.blocks, table, gammas)
    del table
    t_write = time.time() - t0
    pkg = aion_file.parse(data)
    capacity, n_prompt, n_decode = 1024, 128, 511        # the 512-row rings wrap during the decode
    run = PackageRunner(gpu, pkg, capacity=capacity)
    prompt = rng.integers(0, cfg.vocab, n_prompt).astype(np.int32)
    run.run(prompt); run.reset()                         # uploads the weights, builds the prompt's plan
    gpu.sync()
    t = time.perf_counter()
    tok = int(run.run(prompt)["next_token"][0, -1])
    prefill_ms = (time.perf_counter() - t) * 1e3
    if eager:
        gpu.sync()
        t = time.perf_counter()
        for _ in range(32):
            tok = int(run.run(np.array([tok], np.int32))["next_token"][0, -1])
        gpu.sync()
        res = {"steps_decode": run.step_count(1), "eager_tokens": 32, "eager_ms_per_token": round((time.perf_counter() - t) / 32 * 1e3, 4)}
        run.close()
        return res
    run.begin_decode(tok)
    gpu.sync()
    t = time.perf_counter()
    run.decode_run(n_decode)                     # tokens logged on the device, read back once
    gpu.sync()
    decode_s = time.perf_counter() - t
    stream = sum(t_.data.nbytes for t_ in pkg.tensors if t_.quantized)
    res = {"file_bytes": len(data), "nodes": len(pkg.nodes), "write_s": round(t_write, 1),
           "steps_prefill_128": run.step_count(n_prompt), "steps_decode": run.step_count(1),
           "program_nodes": int(gpu.program_node_count(run.program)), "prefill_128_ms": round(prefill_ms, 3),
           "decode_tokens": n_decode, "decode_tokens_per_s": round(n_decode / decode_s, 1),
           "decode_ms_per_token": round(decode_s / n_decode * 1e3, 4), "weight_bytes_per_token": int(stream),
           "weight_GBps": round(stream * n_decode / decode_s / 1e9, 1)}
    run.close()
    return res


def run_decoder(gpu, be, with_cpu=True):
    """BASELINE config 5: 26 layers, hidden 2048, 8 heads / 1 kv head, head_dim 256, GeGLU 8192, vocab 262144,
    q4 weights; 128-token prompt, greedy decode of 128 tokens at batch 1."""
    from aion_amd.decoder import Decoder, DecoderConfig, SyntheticWeights, weight_shapes
    cfg = DecoderConfig()
    t0 = time.time()
    oracle = oracle_alt = None
    if with_cpu:
        from oracle import oracle as orc
        threads = min(16, os.cpu_count() or 1)
        mk = lambda exact: orc.Decoder(cfg.layers, cfg.hidden, cfg.heads, cfg.kv_heads, cfg.head_dim, cfg.ffn, cfg.vocab, cfg.max_seq,
                                       eps=cfg.eps, rope_base=cfg.rope_base, wdtype=cfg.wdtype, threads=threads, attn_exact=exact)
        # the second one differs by one thing (exact exp in attention instead of aion's polynomial): how far the CPU
        # path moves under a 4e-5 perturbation is the yardstick for the GPU's distance from it
        oracle, oracle_alt = mk(False), mk(True)

    def on_weight(name, data):
        oracle.set_weight(name, data)
        oracle_alt.set_weight(name, data)
    dec = Decoder(gpu, cfg, SyntheticWeights(cfg, 0), on_weight=on_weight if oracle else None)
    setup_s = time.time() - t0
    prompt = np.random.default_rng(5).integers(0, cfg.vocab, 128).astype(np.int32)
    weight_bytes = sum(n * k // 32 * 18 for (n, k) in weight_shapes(cfg).values())

    gpu.set_gemm_mode(be.GEMM_BF16_MFMA)
    dec.prefill(prompt); dec.reset()             # warm-up (builds the bf16 weight copies, sizes scratch)
    gpu.sync()
    t = time.perf_counter()
    tok = dec.prefill(prompt)
    prefill_ms = (time.perf_counter() - t) * 1e3
    gpu.set_gemm_mode(be.GEMM_EXACT_I8)
    dec.reset()
    dec.prefill(prompt); dec.reset()
    gpu.sync()
    t = time.perf_counter()
    tok_exact = dec.prefill(prompt)              # the decode continues from the exact-arithmetic prefill
    prefill_exact_ms = (time.perf_counter() - t) * 1e3
    first = tok_exact
    dec.begin_decode(first)
    gpu.sync()
    tokens = []
    t = time.perf_counter()
    for _ in range(128):
        tokens.append(dec.decode_step())
    gpu.sync()
    decode_s = time.perf_counter() - t
    # the same 128 steps without reading the token back each step (device-resident greedy loop)
    dec.pos = 128
    dec.begin_decode(first)
    gpu.sync()
    t = time.perf_counter()
    for _ in range(128):
        dec.decode_step(read_token=False)
    gpu.sync()
    decode_nosync_s = time.perf_counter() - t
    res = {
        "config": "26 layers, hidden 2048, 8q/1kv heads x 256, ffn 8192 (GeGLU), vocab 262144, q4_0 weights, f16 KV cache, prompt 128, greedy 128, batch 1",
        "setup_s": round(setup_s, 1),
        "prefill_128_ms_exact_i8": round(prefill_exact_ms, 3),          # the default mode: aion's arithmetic
        "prefill_tokens_per_s": round(128 / (prefill_exact_ms * 1e-3), 1),
        "prefill_128_ms_bf16_mode": round(prefill_ms, 3),               # bf16 mode keeps the exact kernel at 128 rows (the bf16 one pays from a few hundred on)
        "prefill_next_token_bf16_vs_exact": [int(tok), int(tok_exact)],
        "decode_tokens_per_s": round(128 / decode_s, 1),
        "decode_ms_per_token": round(decode_s / 128 * 1e3, 4),
        "decode_tokens_per_s_no_readback": round(128 / decode_nosync_s, 1),
        "decode_weight_GBps": round(weight_bytes / (decode_nosync_s / 128) / 1e9, 1),
        "weight_bytes_per_token": weight_bytes,
        "program_nodes": int(gpu.program_node_count(dec.program)),
    }
    if oracle is not None:
        # CPU reference-algorithm baseline + parity on a bounded sample: the prompt and 4 decode steps
        t = time.perf_counter()
        otok, ologits = oracle.forward(prompt, 0)
        cpu_prefill_s = time.perf_counter() - t
        atok, alogits = oracle_alt.forward(prompt, 0)
        self_err = float(np.abs(alogits - ologits).max()) / float(np.sqrt((ologits.astype(np.float64) ** 2).mean()))
        dec.reset()
        gtok = dec.prefill(prompt)
        glogits = dec.logits_host()
        rms = float(np.sqrt((ologits.astype(np.float64) ** 2).mean()))
        agree = [int(gtok == otok)]
        errs = [float(np.abs(glogits - ologits).max()) / rms]
        dec.begin_decode(gtok)
        fed = gtok
        t = time.perf_counter()
        n_cpu = 4
        cpu_decode_s = 0.0
        for i in range(n_cpu):
            g_next = dec.decode_step()
            glogits = dec.logits_host()
            t = time.perf_counter()
            o_next, ologits = oracle.forward(np.array([fed], np.int32), 128 + i)
            cpu_decode_s += time.perf_counter() - t
            rms = float(np.sqrt((ologits.astype(np.float64) ** 2).mean()))
            errs.append(float(np.abs(glogits - ologits).max()) / rms)
            agree.append(int(g_next == o_next))
            fed = g_next
        res["cpu_reference"] = {"kind": "port", "cores": min(16, os.cpu_count() or 1),
                                "prefill_128_s": round(cpu_prefill_s, 2), "decode_tokens_per_s": round(n_cpu / cpu_decode_s, 3),
                                "sample": "prompt + %d teacher-forced decode steps" % n_cpu,
                                "gpu_vs_cpu_logits_max_err_over_rms": [round(e, 4) for e in errs],
                                "greedy_token_agreement": agree,
                                "cpu_vs_cpu_exact_exp_logits_max_err_over_rms_prefill": round(self_err, 4),
                                "cpu_vs_cpu_exact_exp_token_agreement_prefill": int(atok == otok),
                                "note": "aion re-quantizes activations to int8 before every matmul: any perturbation flips codes and "
                                        "saturates after a few layers, so the CPU path against itself (exact exp instead of aion's "
                                        "polynomial in attention) moves as far as the GPU is from it"}
    dec.close()
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
        if time.perf_counter() - t0 > 8.0 or reps >= 400:
            break
    dt = time.perf_counter() - t0
    # the same on one thread, on the three smaller shapes (the 302 MB head alone would take seconds per pass)
    t1 = time.perf_counter()
    bytes1, reps1 = 0, 0
    while time.perf_counter() - t1 < 6.0:
        for (n, k) in SHAPES[:3]:
            orc.matmul_q_packed(orc.Q4_0, xs[(n, k)], host_blocks[(n, k)], n, threads=1)
            bytes1 += algorithmic_bytes(18, n, k, batch)
        reps1 += 1
    dt1 = time.perf_counter() - t1
    return {"value": round(total_bytes / dt / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": "%d repetitions of the same four-shape q4 batch-1 step (%.1f s), oracle/aion_oracle.cpp orc_matmul_q_packed "
                      "(aion's packed int8 GEMM at M = 1, kc = 256), -O3 x86-64-v3, threaded over output columns" % (reps, dt),
            "one_thread": {"value": round(bytes1 / dt1 / 1e9, 2), "unit": "GB/s", "cores": 1,
                           "sample": "%d repetitions of the three smaller shapes (%.1f s)" % (reps1, dt1)}}


if __name__ == "__main__":
    main()
