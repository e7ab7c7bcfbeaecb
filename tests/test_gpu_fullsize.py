"""BASELINE config 2's vocabulary-projection shape (N x K = 262144 x 2048) at full size, q4_0 [K,N] and q8_0 [N,K], batch 1 / 4 / 8,
against the CPU oracle - and the persistent row-group loop of every one-row kernel variant on cheap shapes.

This shape is where the one-row kernel runs its largest grid (8192 workgroups), the 2..4-row kernel its persistent grid, and
where 5..8 rows run on the 16-row tile of the exact GEMM at a size no other test reaches. The loop in which a wavefront
walks several row groups (`gwave += wave_stride`, new row addresses, new first loads) starts beyond the grid caps: the
second test enters it with every prologue variant on weights that are long but thin.
Bar: max|err| <= 1e-5 * rms(ref) and the 2e-3 elementwise bound (floored), as for every exact-integer-dot kernel.
"""
import sys

import numpy as np
import pytest

from aion_amd import backend as be
from conftest import norm_err, rms_err, rows_kernel

pytestmark = pytest.mark.gpu
TOL, RMS_TOL = 2e-3, 1e-5
VOCAB_N, VOCAB_K = 262144, 2048


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def tiled_normal(shape, seed, std=0.02):
    """N(0, std) values from a pool tiled to the full size; the pool length is coprime to every row length used here, so no
    two rows or columns of the weight repeat in step with the layout."""
    rng = np.random.default_rng(seed)
    pool = (rng.standard_normal((1 << 22) + 17) * std).astype(np.float32)
    total = int(np.prod(shape))
    return np.tile(pool, -(-total // pool.size))[:total].reshape(shape)


def oracle_rows(orc, dtype, layout, a, blocks, n):
    if layout == be.ROWS_NK:
        return orc.matmul_nt_q8(a, blocks, n, threads=8)
    return orc.matmul_q_packed(dtype, a, blocks, n, threads=8)


@pytest.mark.parametrize("tag,dtype,layout", [("q4", be.Q4_0, be.KMAJOR_KN), ("q8", be.Q8_0, be.ROWS_NK)])
def test_config2_vocabulary_shape_batch_1_4_8(gpu, orc, tag, dtype, layout):
    n, k = VOCAB_N, VOCAB_K
    say("full size", tag, n, k)
    w_f32 = tiled_normal((n, k) if layout == be.ROWS_NK else (k, n), seed=n + k + dtype)
    blocks = be.quantize_blocks(dtype, w_f32, 1 if layout == be.ROWS_NK else 0)
    del w_f32
    w = gpu.upload_weight(dtype, layout, n, k, blocks)
    assert w.packed_bytes == n * k // 32 * be.BLOCK_BYTES[dtype]
    for m in (1, 2, 4, 5, 8):
        a = np.random.default_rng(100 + m).standard_normal((m, k)).astype(np.float32)
        got = gpu.matmul(w, a)
        assert gpu.last_kernel() == ("gemv_%s_fused" % tag if m == 1 else rows_kernel(dtype == be.Q8_0, m, n, k))
        want = oracle_rows(orc, dtype, layout, a, blocks, n)
        e, r = norm_err(got, want), rms_err(got, want)
        say("  m", m, "norm_err", e, "rms_err", r)
        assert e < TOL and r < RMS_TOL, (tag, m, e, r)
    # alpha / beta on a pre-filled C, one row (the epilogue of the strided loop)
    a = np.random.default_rng(7).standard_normal((1, k)).astype(np.float32)
    c0 = np.random.default_rng(8).standard_normal((1, n)).astype(np.float32)
    got = gpu.matmul(w, a, alpha=0.5, beta=-2.0, c=c0)
    want = 0.5 * oracle_rows(orc, dtype, layout, a, blocks, n) - 2.0 * c0
    assert rms_err(got, want) < RMS_TOL
    w.free()


# One row, K = 256, N = 300000 (+ 40003 in the same launch): 75000 row groups of four against a grid capped at 65536
# wavefronts for the plain preparation (512-thread workgroups, eight rounds) and at 8192 for the RMSNorm and gelu-gate
# prologues (256-thread workgroups), so wavefronts take the strided loop - once for some, nine times for others - and with
# two weights in one launch a row group never straddles two weights (the second weight starts mid-grid).
@pytest.mark.parametrize("tag,dtype,layout", [("q4", be.Q4_0, be.KMAJOR_KN), ("q8", be.Q8_0, be.ROWS_NK), ("q8", be.Q8_0, be.KMAJOR_KN)])
def test_strided_row_group_loop_of_every_one_row_variant(gpu, orc, tag, dtype, layout):
    n, n2, k = 300000, 40003, 256
    say("stride path", tag, layout)
    rng = np.random.default_rng(n + dtype + layout)
    made = []
    for nn in (n, n2):
        wf = (rng.standard_normal((nn, k) if layout == be.ROWS_NK else (k, nn)) * 0.05).astype(np.float32)
        blocks = be.quantize_blocks(dtype, wf, 1 if layout == be.ROWS_NK else 0)
        made.append((blocks, gpu.upload_weight(dtype, layout, nn, k, blocks), nn))
    x = rng.standard_normal((1, k)).astype(np.float32)
    xb = gpu.upload(x)
    cs = [gpu.alloc(nn * 4) for _b, _w, nn in made]
    # plain preparation, one weight and two weights
    gpu.step_matmul(made[0][1], xb, 1, cs[0])
    assert gpu.last_kernel() == "gemv_%s_fused" % tag
    want = [oracle_rows(orc, dtype, layout, x, b, nn) for b, _w, nn in made]
    got = gpu.download(cs[0], np.float32, (1, n))
    assert norm_err(got, want[0]) < TOL and rms_err(got, want[0]) < RMS_TOL
    gpu.step_matmul_batch([w for _b, w, _n in made], xb, 1, cs)
    for c, wnt, (_b, _w, nn) in zip(cs, want, made):
        got = gpu.download(c, np.float32, (1, nn))
        assert norm_err(got, wnt) < TOL and rms_err(got, wnt) < RMS_TOL
    # RMSNorm prologue. The norm's sum of squares is reduced in another order than on the CPU, so an activation on a rounding
    # boundary may take the neighbouring int8 code: at K = 256 one flipped code is worth up to ~2e-3 of rms.
    gamma = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    gb = gpu.upload(gamma)
    gpu.step_rmsnorm_matmul([w for _b, w, _n in made], xb, gb, 1, cs, 1e-6)
    assert gpu.last_kernel() == "gemv_%s_rmsnorm" % tag
    h = orc.rmsnorm(x, gamma, 1e-6)
    for c, (b, _w, nn) in zip(cs, made):
        got = gpu.download(c, np.float32, (1, nn))
        assert rms_err(got, oracle_rows(orc, dtype, layout, h, b, nn)) < 6e-3
    # gelu-gate prologue (one weight), accumulating into C
    gate = (rng.standard_normal((1, k)) * 2).astype(np.float32)
    up = rng.standard_normal((1, k)).astype(np.float32)
    c0 = rng.standard_normal((1, n)).astype(np.float32)
    gtb, upb, cb = gpu.upload(gate), gpu.upload(up), gpu.upload(c0)
    gpu.step_gate_matmul(made[0][1], gtb, upb, 1, cb, beta=1.0)
    assert gpu.last_kernel() == "gemv_%s_gate" % tag
    act = orc.gate_gelu(gate, up).reshape(1, k)
    want_g = oracle_rows(orc, dtype, layout, act, made[0][0], n) + c0
    assert rms_err(gpu.download(cb, np.float32, (1, n)), want_g) < 6e-3
    for t in [xb, gb, gtb, upb, cb] + cs:
        t.free()
    for _b, w, _n in made:
        w.free()


# The fused GeGLU block with more quant blocks of hidden activations (F / 32 = 2100) than the gate/up kernel has workgroups
# (8 per CU = 2048 on 256 CUs): its workgroups walk a second task, re-using the LDS slots of the first.
@pytest.mark.parametrize("tag,dtype", [("q4", be.Q4_0), ("q8", be.Q8_0)])
def test_geglu_block_with_more_tasks_than_workgroups(gpu, orc, tag, dtype):
    k, f = 256, 2100 * 32
    say("geglu stride path", tag)
    rng = np.random.default_rng(f + dtype)
    mk = lambda n, kk, std: be.quantize_blocks(dtype, (rng.standard_normal((kk, n)) * std).astype(np.float32), 0)
    bg, bu, bd = mk(f, k, 0.05), mk(f, k, 0.05), mk(k, f, 0.02)
    wg, wu, wd = (gpu.upload_weight(dtype, be.KMAJOR_KN, n, kk, b) for (n, kk, b) in ((f, k, bg), (f, k, bu), (k, f, bd)))
    x = rng.standard_normal((1, k)).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    xb, gb = gpu.upload(x), gpu.upload(gamma)
    gpu.step_rmsnorm_geglu_matmul(wg, wu, wd, xb, gb, 1e-6, xb, beta=1.0)            # x += down(gelu(gate) * up)
    got = gpu.download(xb, np.float32, (1, k))
    h = orc.rmsnorm(x, gamma, 1e-6)
    g = orc.matmul_q_packed(dtype, h, bg, f, threads=8)
    u = orc.matmul_q_packed(dtype, h, bu, f, threads=8)
    want = orc.matmul_q_packed(dtype, orc.gate_gelu(g, u).reshape(1, f), bd, k, beta=1.0, c=x, threads=8)
    # flipped int8 codes of the normalised row move g and u by ~1e-3; the long down projection averages that out
    assert rms_err(got, want) < 3e-3, rms_err(got, want)
    # and against the same block as separate steps on the device (the same prepared codes up to such flips)
    x2, g2, u2 = gpu.upload(x), gpu.alloc(f * 4), gpu.alloc(f * 4)
    gpu.step_rmsnorm_matmul([wg, wu], x2, gb, 1, [g2, u2], 1e-6)
    gpu.step_gate_matmul(wd, g2, u2, 1, x2, beta=1.0)
    sep = gpu.download(x2, np.float32, (1, k))
    assert rms_err(got, sep) < 2e-3
    for t in (xb, gb, x2, g2, u2):
        t.free()
    for w in (wg, wu, wd):
        w.free()
