"""GPU parity of the prefill GEMM paths (BASELINE config 3) against the CPU oracle.

EXACT_I8: same arithmetic as aion's CPU kernels (int8 activations, exact block dots): held to
max|err| <= 1e-5 rms(ref) and the 2e-3 elementwise bound. BF16_MFMA: weights dequantized to
bf16, activations rounded to bf16, f32 accumulate: normalised error <= 1e-2 against the
f32-activation dequant oracle and NMSE <= 1e-4 against the int8-activation CPU oracle (the
activation-quantization noise floor is ~3e-5). Rows of A never interact, so at the full
config-3 sizes the oracle is evaluated on a sample of rows.
"""
import sys

import numpy as np
import pytest

from aion_amd import backend as be
from conftest import norm_err, rms_err

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def bf16_round(a):
    """f32 -> nearest-even bf16, returned as f32 (config 3: activations are cast to bf16 for the MFMA path)"""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint32) << 16).view(np.float32)


CASES = [(be.Q8_0, be.ROWS_NK), (be.Q8_0, be.KMAJOR_KN), (be.Q4_0, be.KMAJOR_KN)]


def make_weight(gpu, dtype, layout, n, k, seed):
    rng = np.random.default_rng(seed)
    shape = (n, k) if layout == be.ROWS_NK else (k, n)
    w = (rng.standard_normal(shape) * 0.02).astype(np.float32)
    blocks = be.quantize_blocks(dtype, w, 1 if layout == be.ROWS_NK else 0)
    return blocks, gpu.upload_weight(dtype, layout, n, k, blocks)


def oracle_i8(orc, dtype, layout, a, blocks, n, **kw):
    if layout == be.ROWS_NK:
        return orc.matmul_nt_q8(a, blocks, n, threads=8, **kw)
    return orc.matmul_q_packed(dtype, a, blocks, n, threads=8, **kw)


@pytest.mark.parametrize("dtype,layout", CASES)
@pytest.mark.parametrize("m,n,k", [(9, 64, 64), (17, 100, 96), (33, 300, 256), (70, 257, 512), (130, 1000, 1024)])
def test_exact_gemm_ragged_shapes(gpu, orc, dtype, layout, m, n, k):
    say("exact", dtype, layout, m, n, k)
    gpu.set_gemm_mode(be.GEMM_EXACT_I8)
    blocks, w = make_weight(gpu, dtype, layout, n, k, seed=m + n + k)
    a = np.random.default_rng(m).standard_normal((m, k)).astype(np.float32)
    a[0, :32] = 0
    got = gpu.matmul(w, a)
    assert gpu.last_kernel() == ("gemm_i8_q8" if dtype == be.Q8_0 else "gemm_i8_q4")
    want = oracle_i8(orc, dtype, layout, a, blocks, n)
    assert norm_err(got, want) < 2e-3 and rms_err(got, want) < 1e-5, (norm_err(got, want), rms_err(got, want))
    # alpha / beta
    c0 = np.random.default_rng(1).standard_normal((m, n)).astype(np.float32)
    got2 = gpu.matmul(w, a, alpha=0.5, beta=2.0, c=c0)
    want2 = oracle_i8(orc, dtype, layout, a, blocks, n, alpha=0.5, beta=2.0, c=c0)
    assert rms_err(got2, want2) < 1e-5
    w.free()


@pytest.mark.parametrize("dtype,layout", CASES)
def test_exact_gemm_rows_match_decode_path(gpu, orc, dtype, layout):
    # the GEMM and the GEMV compute the same formula: per-row results agree to f32 summation order
    gpu.set_gemm_mode(be.GEMM_EXACT_I8)
    blocks, w = make_weight(gpu, dtype, layout, 512, 1024, seed=3)
    a = np.random.default_rng(4).standard_normal((40, 1024)).astype(np.float32)
    full = gpu.matmul(w, a)
    one = gpu.matmul(w, a[7:8])
    assert rms_err(full[7:8], one) < 1e-5
    w.free()


# every (M, N) pair of config 3 (each picks its own tile and launch shape) in every weight format and layout
@pytest.mark.parametrize("dtype,layout", CASES)
@pytest.mark.parametrize("m,n", [(512, 4096), (512, 14336), (2048, 4096), (2048, 14336)])
def test_config3_exact_full_size_on_row_sample(gpu, orc, dtype, layout, m, n):
    k = 4096
    say("config3 exact", dtype, m, n)
    gpu.set_gemm_mode(be.GEMM_EXACT_I8)
    blocks, w = make_weight(gpu, dtype, layout, n, k, seed=n)
    a = np.random.default_rng(m).standard_normal((m, k)).astype(np.float32)
    got = gpu.matmul(w, a)
    rows = np.array([0, 1, 15, 16, 63, 64, m // 2 + 3, m - 2, m - 1])
    want = oracle_i8(orc, dtype, layout, np.ascontiguousarray(a[rows]), blocks, n)
    assert norm_err(got[rows], want) < 2e-3 and rms_err(got[rows], want) < 1e-5
    w.free()


@pytest.mark.parametrize("dtype,layout", CASES)
@pytest.mark.parametrize("m,n,k", [(9, 64, 64), (100, 130, 256), (300, 520, 1024)])
def test_bf16_gemm_ragged_shapes(gpu, orc, dtype, layout, m, n, k):
    say("bf16", dtype, layout, m, n, k)
    gpu.set_gemm_mode(be.GEMM_BF16_MFMA_ALWAYS)         # shapes this small run on the exact kernel in the plain bf16 mode
    try:
        blocks, w = make_weight(gpu, dtype, layout, n, k, seed=m * n)
        a = bf16_round(np.random.default_rng(k).standard_normal((m, k)).astype(np.float32))
        got = gpu.matmul(w, a)
        assert gpu.last_kernel() == "gemm_bf16"
        f32a = orc.matmul_q_f32a(dtype, layout == be.ROWS_NK, a, blocks, n, threads=8)
        e = norm_err(got, f32a)
        say("  norm err vs f32-A", e)
        # the dequantized weight is rounded to bf16 (relative error <= 2^-8 per product, random sign):
        # the output error is ~1.6e-3 of rms(ref) at 1 sigma, independent of k
        assert rms_err(got, f32a) < 1e-2
        i8 = oracle_i8(orc, dtype, layout, a, blocks, n)
        nmse = float(((got - i8) ** 2).sum() / (i8 ** 2).sum())
        assert nmse < 1e-4
        c0 = np.random.default_rng(2).standard_normal((m, n)).astype(np.float32)
        got2 = gpu.matmul(w, a, alpha=0.5, beta=2.0, c=c0)
        assert np.allclose(got2, 0.5 * got + 2.0 * c0, rtol=1e-5, atol=1e-5)
        w.free()
    finally:
        gpu.set_gemm_mode(be.GEMM_EXACT_I8)


# (2048, 14336): 32 column tiles of 256 and 32 of 192 interleaved in one launch (wide, wide, narrow, narrow, ...);
# (2048, 13000): 32 of 256 and 26 of 192 - thirteen whole blocks of that pattern, then the rest of the wide tiles; the last
# narrow tile hangs over the last column. (2048, 9092): 48 tiles of 192 only (two rounds of 3/4 beat one wide round plus a
# narrow one), the last one hanging over; (2048, 5120): 27 tiles of 192 in one round instead of two rounds of 128-row tiles.
# (1300, 11008): 258 tiles of 256 rows would need a second round, so 473 tiles of 128 rows run in two half-time rounds.
# Rows from every 256-row tile, all columns.
@pytest.mark.parametrize("dtype,layout", CASES)
@pytest.mark.parametrize("m,n", [(512, 4096), (512, 14336), (2048, 4096), (2048, 14336), (2048, 9092), (2048, 13000), (2048, 5120), (1300, 11008)])
def test_config3_bf16_full_size_on_row_sample(gpu, orc, dtype, layout, m, n):
    k = 4096
    say("config3 bf16", dtype, m, n)
    gpu.set_gemm_mode(be.GEMM_BF16_MFMA_ALWAYS)
    try:
        blocks, w = make_weight(gpu, dtype, layout, n, k, seed=n + 1)
        a = bf16_round(np.random.default_rng(m + 1).standard_normal((m, k)).astype(np.float32))
        got = gpu.matmul(w, a)
        rows = np.unique(np.array([0, 17, 255, 256, m // 2, m - 1] + [t * 256 + 29 * (t + 1) for t in range(m // 256)]))
        f32a = orc.matmul_q_f32a(dtype, layout == be.ROWS_NK, np.ascontiguousarray(a[rows]), blocks, n, threads=8)
        r = rms_err(got[rows], f32a)
        say("  max|err|/rms vs f32-A dequant", r)
        assert r < 1e-2
        i8 = oracle_i8(orc, dtype, layout, np.ascontiguousarray(a[rows]), blocks, n)
        assert float(((got[rows] - i8) ** 2).sum() / (i8 ** 2).sum()) < 1e-4
        w.free()
    finally:
        gpu.set_gemm_mode(be.GEMM_EXACT_I8)


@pytest.mark.parametrize("dtype,layout", CASES)
def test_exact_gemm_k_slices(gpu, orc, dtype, layout):
    """Few workgroups against a long K: the exact kernel cuts the K steps into slices across workgroups (grid z) and a
    second launch adds the slices in order. Parity as for every exact kernel, alpha / beta / row pitch through the second
    launch, the same bits on a second run (nothing depends on which slice finishes first), and sibling weights that share
    the launch."""
    say("k slices", dtype, layout)
    m, n, k = 24, 520, 8192
    gpu.set_gemm_mode(be.GEMM_EXACT_I8)
    blocks, w = make_weight(gpu, dtype, layout, n, k, seed=41)
    blocks2, w2 = make_weight(gpu, dtype, layout, 200, k, seed=42)
    rng = np.random.default_rng(43)
    a = rng.standard_normal((m, k)).astype(np.float32)
    a_buf = gpu.upload(a)
    ldc = 524
    c0 = rng.standard_normal((m, ldc)).astype(np.float32)
    c_buf = gpu.upload(c0)
    gpu.profile_start()
    gpu.step_matmul(w, a_buf, m, c_buf, ldc=ldc, alpha=0.5, beta=2.0)
    prof = gpu.profile_stop()
    assert [nm for nm, _ in prof if nm.startswith("gemm_i8")] == [prof[-1][0]] * 2        # the sliced kernel and the fold
    got = gpu.download(c_buf, np.float32, (m, ldc))
    want = oracle_i8(orc, dtype, layout, a, blocks, n, alpha=0.5, beta=2.0, c=np.ascontiguousarray(c0[:, :n]))
    assert norm_err(got[:, :n], want) < 2e-3 and rms_err(got[:, :n], want) < 1e-5
    assert np.array_equal(got[:, n:], c0[:, n:])
    first = gpu.matmul(w, a)
    assert np.array_equal(first.view(np.uint32), gpu.matmul(w, a).view(np.uint32))
    c1, c2 = gpu.alloc(m * n * 4), gpu.alloc(m * 200 * 4)
    gpu.step_matmul_batch([w, w2], a_buf, m, [c1, c2])
    got1, got2 = gpu.download(c1, np.float32, (m, n)), gpu.download(c2, np.float32, (m, 200))
    assert rms_err(got1, oracle_i8(orc, dtype, layout, a, blocks, n)) < 1e-5
    assert rms_err(got2, oracle_i8(orc, dtype, layout, a, blocks2, 200)) < 1e-5
    for t in (a_buf, c_buf, c1, c2):
        t.free()
    w.free(); w2.free()


@pytest.mark.parametrize("dtype,layout", CASES)
@pytest.mark.parametrize("m,n,k", [(2048, 14336, 4096), (512, 4096, 4096), (300, 520, 1056), (1300, 11008, 4096), (70, 200, 96)])
def test_bf16_gemm_without_weight_copies_gives_the_same_bits(gpu, orc, dtype, layout, m, n, k):
    """The bf16 kernel's two weight operands: the bf16 copy the context keeps of a weight, and the weight's quant blocks
    converted while the kernel stages them (aionhip_set_bf16_weight_copies(0): nothing resident, nothing allocated).
    Both round code * scale to bf16 once and multiply in the same order: the same bits, every tile shape (256 x 256 and
    256 x 192 mixed, 128-row, 64-row and 64 x 128 tiles, ragged edges, a K that is not a multiple of four blocks)."""
    say("bf16 without copies", dtype, layout, m, n, k)
    gpu.set_gemm_mode(be.GEMM_BF16_MFMA_ALWAYS)
    try:
        blocks, w = make_weight(gpu, dtype, layout, n, k, seed=m + n)
        a = bf16_round(np.random.default_rng(k).standard_normal((m, k)).astype(np.float32))
        copies0 = gpu.bf16_copy_stats()
        with_copy = gpu.matmul(w, a)
        assert gpu.last_kernel() == "gemm_bf16" and gpu.bf16_copy_stats()[0] == copies0[0] + 1
        w.drop_bf16()
        assert gpu.bf16_copy_stats() == copies0
        gpu.set_bf16_weight_copies(False)
        streamed = gpu.matmul(w, a)
        assert gpu.last_kernel() == "gemm_bf16" and gpu.bf16_copy_stats() == copies0      # no copy was built
        assert np.array_equal(with_copy.view(np.uint32), streamed.view(np.uint32))
        rows = np.unique(np.array([0, m // 3, m - 1]))
        f32a = orc.matmul_q_f32a(dtype, layout == be.ROWS_NK, np.ascontiguousarray(a[rows]), blocks, n, threads=8)
        assert rms_err(streamed[rows], f32a) < 1e-2
        c0 = np.random.default_rng(2).standard_normal((m, n)).astype(np.float32)
        got2 = gpu.matmul(w, a, alpha=0.5, beta=2.0, c=c0)
        assert np.allclose(got2, 0.5 * streamed + 2.0 * c0, rtol=1e-5, atol=1e-5)
        w.free()
    finally:
        gpu.set_bf16_weight_copies(True)
        gpu.set_gemm_mode(be.GEMM_EXACT_I8)


@pytest.mark.parametrize("ldc,c_offset", [(520, 0), (524, 0), (521, 0), (528, 3)])
def test_bf16_gemm_alpha_beta_and_output_strides(gpu, orc, ldc, c_offset):
    """The bf16 kernel's epilogue: 16-byte stores where the output rows allow them (row pitch and base 16-byte aligned),
    single floats otherwise (odd pitch, a base that is only 4-byte aligned), alpha and beta in both, the columns between
    n and the pitch untouched. Checked against the same kernel's plain product: C' = alpha * (A W^T) + beta * C."""
    say("bf16 alpha/beta", ldc, c_offset)
    m, n, k = 300, 520, 1024
    gpu.set_gemm_mode(be.GEMM_BF16_MFMA_ALWAYS)
    try:
        blocks, w = make_weight(gpu, be.Q4_0, be.KMAJOR_KN, n, k, seed=31)
        rng = np.random.default_rng(32)
        a = rng.standard_normal((m, k)).astype(np.float32)
        c0 = rng.standard_normal(m * ldc + c_offset).astype(np.float32)
        plain = gpu.matmul(w, a)
        assert gpu.last_kernel() == "gemm_bf16"
        a_buf, c_buf = gpu.upload(a), gpu.upload(c0)
        gpu.step_matmul(w, a_buf, m, c_buf, ldc=ldc, alpha=0.5, beta=2.0, c_offset=c_offset * 4)
        got = gpu.download(c_buf, np.float32, (m * ldc + c_offset,))
        assert np.array_equal(got[:c_offset], c0[:c_offset])
        got2, old2 = got[c_offset:].reshape(m, ldc), c0[c_offset:].reshape(m, ldc)
        want = 0.5 * plain + 2.0 * old2[:, :n]
        assert float(np.abs(got2[:, :n] - want).max()) <= 1e-5 * float(np.abs(want).max())
        assert np.array_equal(got2[:, n:], old2[:, n:])
        a_buf.free(); c_buf.free(); w.free()
    finally:
        gpu.set_gemm_mode(be.GEMM_EXACT_I8)


def test_bf16_mode_runs_the_bf16_kernel_only_where_it_pays(gpu, orc):
    """In bf16 mode a shape the bf16 kernel is not expected to win (few rows: it streams a 2-byte copy of the weight
    through 256-column tiles) stays on the exact kernel - same numbers as the exact mode - and a large one moves."""
    blocks, w = make_weight(gpu, be.Q4_0, be.KMAJOR_KN, 4096, 4096, seed=5)
    rng = np.random.default_rng(6)
    small, large = rng.standard_normal((48, 4096)).astype(np.float32), rng.standard_normal((2048, 4096)).astype(np.float32)
    exact_small = gpu.matmul(w, small)
    gpu.set_gemm_mode(be.GEMM_BF16_MFMA)
    try:
        got = gpu.matmul(w, small)
        assert gpu.last_kernel() == "gemm_i8_q4" and np.array_equal(got, exact_small)
        gpu.matmul(w, large)
        assert gpu.last_kernel() == "gemm_bf16"
        gpu.set_gemm_mode(be.GEMM_BF16_MFMA_ALWAYS)
        gpu.matmul(w, small)
        assert gpu.last_kernel() == "gemm_bf16"
    finally:
        gpu.set_gemm_mode(be.GEMM_EXACT_I8)
    w.free()
