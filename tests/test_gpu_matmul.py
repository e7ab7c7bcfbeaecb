"""GPU parity of the quantized matmul steps against the CPU oracle (through the C ABI).

Tolerance: the north-star bound for f32-accumulate kernels is max relative error 2e-3, taken
elementwise with a floor (conftest.norm_err). The integer block dots are exact here, so only the
f32 summation order differs: the tests additionally hold max|err| to 1e-5 of rms(ref)
(conftest.rms_err). Block bytes are compared bit-exactly.
"""
import sys

import numpy as np
import pytest

from aion_amd import backend as be
from aion_amd import hip
from conftest import norm_err, rms_err, rows_kernel

pytestmark = pytest.mark.gpu
TOL = 2e-3      # elementwise, floored
RMS_TOL = 1e-5  # max |err| / rms(ref)


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def make_weight(gpu, orc, dtype, layout, n, k, seed, std=0.02):
    rng = np.random.default_rng(seed)
    if layout == be.ROWS_NK:
        w = (rng.standard_normal((n, k)) * std).astype(np.float32)
        blocks = be.quantize_blocks(dtype, w, 1)
    else:
        w = (rng.standard_normal((k, n)) * std).astype(np.float32)
        blocks = be.quantize_blocks(dtype, w, 0)
    return blocks, gpu.upload_weight(dtype, layout, n, k, blocks)


def oracle_matmul(orc, dtype, layout, a, blocks, n, **kw):
    if layout == be.ROWS_NK:
        return orc.matmul_nt_q8(a, blocks, n, threads=8, **kw)
    if dtype == be.Q8_0 and a.shape[0] <= 16:
        return orc.matmul_q8_kmajor(a, blocks, n, threads=8, **kw)
    return orc.matmul_q_packed(dtype, a, blocks, n, threads=8, **kw)


CASES = [(be.Q8_0, be.ROWS_NK), (be.Q8_0, be.KMAJOR_KN), (be.Q4_0, be.KMAJOR_KN)]


@pytest.mark.parametrize("dtype,layout", CASES)
def test_weight_relay_is_a_byte_permutation(gpu, orc, dtype, layout):
    say("relay", dtype, layout)
    for n, k in [(5, 64), (64, 2048), (33, 160)]:
        blocks, w = make_weight(gpu, orc, dtype, layout, n, k, seed=n * k)
        assert w.packed_bytes == blocks.nbytes
        assert np.array_equal(w.download(), blocks)
        w.free()


def test_weight_upload_with_block_row_stride(gpu, orc):
    # MatMulParams.ldb: a [K,N] view whose block rows are ld blocks apart
    n, k, ld = 6, 96, 10
    rng = np.random.default_rng(0)
    full = (rng.standard_normal((k, ld)) * 0.02).astype(np.float32)
    packed_full = be.quantize_blocks(be.Q8_0, full, 0)                     # [k/32, ld] blocks
    compact = be.quantize_blocks(be.Q8_0, np.ascontiguousarray(full[:, :n]), 0)
    w_strided = gpu.upload_weight(be.Q8_0, be.KMAJOR_KN, n, k, packed_full, ld_blocks=ld)
    w_compact = gpu.upload_weight(be.Q8_0, be.KMAJOR_KN, n, k, compact)
    a = rng.standard_normal((2, k)).astype(np.float32)
    # aion cpu/test_cpu_kernels.zig:726-825: strided sub-block == compact copy, bit-exactly
    assert np.array_equal(gpu.matmul(w_strided, a), gpu.matmul(w_compact, a))
    assert np.array_equal(w_strided.download(), compact)
    w_strided.free(); w_compact.free()


@pytest.mark.parametrize("dtype", [be.Q8_0, be.Q4_0])
@pytest.mark.parametrize("axis", [0, 1])
def test_device_quantizer_bytes_match_oracle(gpu, orc, dtype, axis):
    say("device quantizer", dtype, axis)
    rng = np.random.default_rng(17 + axis)
    rows, cols = (96, 40) if axis == 0 else (40, 96)
    v = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32)
    v[0:32, 0] = 0.0
    v[0, 0:32] = 0.0
    v.reshape(-1)[5] = 0.5            # large outlier
    # a block whose codes depend on WHICH scale divides (q4: the f32 scale; q8: the f16-rounded one), by hand:
    # max_abs = 7 * (1 + 2^-12) -> q4 codes 7, 2, -2, 0 for 2.5, -2.5, 0.5 (3, -3, 1 if the stored f16 scale 1.0 divided)
    special = np.zeros(32, np.float32)
    special[:4] = [7.0 + 7.0 / 4096.0, 2.5, -2.5, 0.5]
    if axis == 0:
        v[32:64, 3] = special
    else:
        v[3, 32:64] = special
    src = gpu.upload(v)
    dst = gpu.quantize_device(dtype, src, rows, cols, axis)
    got = gpu.download(dst, np.uint8)
    assert np.array_equal(got, orc.quantize(dtype, v, axis))
    src.free(); dst.free()


@pytest.mark.parametrize("dtype,layout", CASES)
@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 8])
def test_gemv_small_and_ragged_shapes(gpu, orc, dtype, layout, m):
    for n, k in [(1, 32), (5, 64), (13, 160), (67, 2080), (256, 1024)]:
        say("gemv small", dtype, layout, m, n, k)
        blocks, w = make_weight(gpu, orc, dtype, layout, n, k, seed=n + k + m, std=0.5)
        a = np.random.default_rng(m * 31 + n).standard_normal((m, k)).astype(np.float32)
        a[0, :32] = 0.0                                       # a zero activation block (scale 0)
        got = gpu.matmul(w, a)
        want = oracle_matmul(orc, dtype, layout, a, blocks, n)
        assert norm_err(got, want) < TOL and rms_err(got, want) < RMS_TOL, (n, k, norm_err(got, want), rms_err(got, want))
        want_kernel = "gemv_q8" if dtype == be.Q8_0 else "gemv_q4"
        assert gpu.last_kernel() == (want_kernel + "_fused" if m == 1 else want_kernel)
        w.free()


def test_config1_q8_gemv_2048(gpu, orc):
    # BASELINE config 1: W 2048x2048 ~N(0,0.02) -> q8 (aion's quantizer), x ~N(0,1), y = W.x
    say("config1")
    blocks, w = make_weight(gpu, orc, be.Q8_0, be.ROWS_NK, 2048, 2048, seed=1)
    x = np.random.default_rng(2).standard_normal((1, 2048)).astype(np.float32)
    got = gpu.matmul(w, x)
    want = orc.matmul_nt_q8(x, blocks, 2048)
    assert norm_err(got, want) < TOL and rms_err(got, want) < RMS_TOL
    # and against the f32-activation dequant family: differs by activation-quant noise only
    f32a = orc.matmul_q_f32a(orc.Q8_0, True, x, blocks, 2048)
    nmse = float(((got - f32a) ** 2).sum() / (f32a ** 2).sum())
    assert nmse < 2e-4
    w.free()


def test_reference_closed_form_kmajor_past_8192(gpu, orc):
    # aion cpu/kernels/matvec_q.zig:176-219 inputs (m=2, n=5, k=8192+64), rel 1e-5 there
    m, n, k = 2, 5, 8192 + 64
    kb = k // 32
    a = (((np.arange(m * k) % 37) - 18) * 0.01).astype(np.float32).reshape(m, k)
    blocks = np.zeros((kb * n, 34), np.uint8)
    blocks[:, 0:2] = np.array([0.02], np.float16).view(np.uint8)
    bi = np.arange(kb * n, dtype=np.uint64)[:, None]
    t = np.arange(32, dtype=np.uint64)[None, :]
    blocks[:, 2:] = ((bi * np.uint64(5) + t * np.uint64(3)) & np.uint64(0xFF)).astype(np.uint8)
    w = gpu.upload_weight(be.Q8_0, be.KMAJOR_KN, n, k, blocks)
    got = gpu.matmul(w, a)
    want = orc.matmul_q8_kmajor(a, blocks, n)
    assert np.allclose(got, want, rtol=1e-5, atol=0)
    w.free()


@pytest.mark.parametrize("dtype,layout", CASES)
def test_alpha_beta_and_strides(gpu, orc, dtype, layout):
    say("alpha/beta", dtype, layout)
    m, n, k, lda, ldc = 3, 37, 96, 128, 50
    blocks, w = make_weight(gpu, orc, dtype, layout, n, k, seed=9, std=0.3)
    rng = np.random.default_rng(10)
    a_full = rng.standard_normal((m, lda)).astype(np.float32)
    c_full = rng.standard_normal((m, ldc)).astype(np.float32)
    a_buf, c_buf = gpu.upload(a_full), gpu.upload(c_full)
    gpu.step_matmul(w, a_buf, m, c_buf, lda=lda, ldc=ldc, alpha=0.5, beta=2.0)
    got = gpu.download(c_buf, np.float32, (m, ldc))
    a = np.ascontiguousarray(a_full[:, :k])
    want = oracle_matmul(orc, dtype, layout, a, blocks, n, alpha=0.5, beta=2.0, c=np.ascontiguousarray(c_full[:, :n]))
    assert norm_err(got[:, :n], want) < TOL and rms_err(got[:, :n], want) < RMS_TOL
    assert np.array_equal(got[:, n:], c_full[:, n:])           # padding columns untouched
    a_buf.free(); c_buf.free(); w.free()


@pytest.mark.parametrize("dtype,layout", CASES)
@pytest.mark.parametrize("n,k", [(4096, 4096), (14336, 4096), (4096, 14336)])
def test_config2_decode_shapes(gpu, orc, dtype, layout, n, k):
    # BASELINE config 2 shapes at batch 1, 4, 8 (the 262144x2048 shape is in test_gpu_fullsize.py)
    say("config2", dtype, layout, n, k)
    blocks, w = make_weight(gpu, orc, dtype, layout, n, k, seed=n ^ k)
    for m in (1, 4, 8):
        a = np.random.default_rng(m).standard_normal((m, k)).astype(np.float32)
        got = gpu.matmul(w, a)
        want = oracle_matmul(orc, dtype, layout, a, blocks, n)
        e, r = norm_err(got, want), rms_err(got, want)
        say("  m", m, "norm_err", e, "rms_err", r)
        assert e < TOL and r < RMS_TOL
    w.free()


# One activation row against a long reduction axis: past K = 4096 the K axis is cut into slices across workgroups, each of
# which prepares its own slice of the activation (gemv_ksplit_kernel); past 65536 columns or rows the activation is prepared
# by a launch of its own and the GEMV reads it from memory. Up to K = 8192 a weight of 16384 or more outputs stays on the
# kernel that prepares the whole activation in every workgroup (the weight stream hides the prologue). Edges: the first K past 4096, few rows and one row, K that is not
# a multiple of the 64 chunks a wavefront covers per pass or of the slice count, the config-2 shape 4096 x 14336, alpha/beta.
# The last four: row pitches of 4, 8 and 32 KiB, where the workgroups take the slices in alternating instead of slice-major
# order (q8 8192 and 32768, q4 8192 and 16384).
@pytest.mark.parametrize("dtype,layout", CASES)
@pytest.mark.parametrize("n,k,kernel", [(5, 4128, "ksplit"), (300, 16384, "ksplit"), (70, 16416, "ksplit"), (2050, 8224, "ksplit"), (9000, 4096, "fused"),
                                        (4096, 14336, "ksplit"), (1, 32768, "ksplit"), (33, 65568, "gemv"), (70000, 4128, "fused"),
                                        (16390, 8192, "fused"), (16376, 8192, "ksplit"), (66000, 8224, "gemv"),
                                        (4100, 8192, "ksplit"), (8200, 8192, "ksplit"), (4100, 16384, "ksplit"), (40, 32768, "ksplit")])
def test_single_row_long_k(gpu, orc, dtype, layout, n, k, kernel):
    say("single row, long k", dtype, layout, n, k)
    blocks, w = make_weight(gpu, orc, dtype, layout, n, k, seed=n + k)
    a = np.random.default_rng(k).standard_normal((1, k)).astype(np.float32)
    got = gpu.matmul(w, a)
    q = "q8" if dtype == be.Q8_0 else "q4"
    assert gpu.last_kernel() == {"fused": "gemv_%s_fused", "ksplit": "gemv_%s_ksplit", "gemv": "gemv_%s"}[kernel] % q
    want = oracle_matmul(orc, dtype, layout, a, blocks, n)
    assert norm_err(got, want) < TOL and rms_err(got, want) < RMS_TOL
    if kernel == "ksplit":
        # the partial sums of the K slices meet along a fixed tree: the same bits on every run, whichever workgroup is last
        for _ in range(3):
            assert np.array_equal(gpu.matmul(w, a), got)
    c0 = np.random.default_rng(1).standard_normal((1, n)).astype(np.float32)
    got2 = gpu.matmul(w, a, alpha=0.5, beta=-2.0, c=c0)
    want2 = oracle_matmul(orc, dtype, layout, a, blocks, n, alpha=0.5, beta=-2.0, c=c0)
    assert norm_err(got2, want2) < TOL and rms_err(got2, want2) < RMS_TOL
    w.free()


def test_last_launch_names_the_kernel_instance_and_its_grid(gpu, orc):
    """What reports print beside a figure so that it can be matched to a kernel trace: the instance's name as a trace prints
    it (template arguments included, no parameter list), the grid in workgroups, the workgroup size, the dynamic LDS bytes."""
    n, k = 4096, 4096
    blocks, w = make_weight(gpu, orc, be.Q4_0, be.KMAJOR_KN, n, k, seed=3)
    gpu.matmul(w, np.ones((1, k), np.float32))
    ll = gpu.last_launch()
    say("last_launch", ll)
    assert gpu.last_kernel() == "gemv_q4_fused"
    assert "gemv_fused_kernel<" in ll["kernel"] and ll["kernel"].endswith(">") and "(" not in ll["kernel"].replace("(anonymous namespace)", "")
    assert ll["block"] == [1024, 1, 1] and ll["grid"][1:] == [1, 1] and 1 <= ll["grid"][0] <= n // 8
    assert ll["lds"] >= k + k // 32 * 8
    w.free()


def test_single_row_q4_eight_alternating_slices(gpu, orc):
    # q4 at K = 65536: eight slices over a row pitch of 32 KiB, taken in alternating order
    n, k = 24, 65536
    blocks, w = make_weight(gpu, orc, be.Q4_0, be.KMAJOR_KN, n, k, seed=5)
    a = np.random.default_rng(5).standard_normal((1, k)).astype(np.float32)
    got = gpu.matmul(w, a)
    assert gpu.last_kernel() == "gemv_q4_ksplit"
    want = oracle_matmul(orc, be.Q4_0, be.KMAJOR_KN, a, blocks, n)
    assert norm_err(got, want) < TOL and rms_err(got, want) < RMS_TOL
    assert np.array_equal(gpu.matmul(w, a), got)
    w.free()


# Sibling weights at 3..8 rows whose rows together reach the matrix-pipe GEMV's range (gate / up of a feed-forward block, a short
# prompt): one launch walks the tiles of all weights; ragged column counts, a sibling far smaller than the others, alpha / beta.
@pytest.mark.parametrize("dtype,m,ns,k", [(be.Q4_0, 6, (8200, 8192), 2048), (be.Q4_0, 5, (14000, 40, 1000), 4096), (be.Q4_0, 3, (40000, 30000), 2304),
                                          (be.Q8_0, 4, (33000, 33000), 2048)])
def test_sibling_weights_share_a_matrix_pipe_gemv_launch(gpu, orc, dtype, m, ns, k):
    say("sibling gemv mfma", dtype, m, ns, k)
    layout = be.ROWS_NK if dtype == be.Q8_0 else be.KMAJOR_KN
    made = [make_weight(gpu, orc, dtype, layout, n, k, seed=n + 3 * i, std=0.1) for i, n in enumerate(ns)]
    rng = np.random.default_rng(m + k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    c0 = [rng.standard_normal((m, n)).astype(np.float32) for n in ns]
    a_buf = gpu.upload(a)
    for alpha, beta in ((1.0, 0.0), (-0.5, 1.5)):
        c_bufs = [gpu.upload(c) for c in c0]
        gpu.profile_start()
        gpu.step_matmul_batch([w for _b, w in made], a_buf, m, c_bufs, alpha=alpha, beta=beta)
        names = [nm for nm, _ms in gpu.profile_stop()]
        assert names.count("gemv_%s_mfma" % ("q8" if dtype == be.Q8_0 else "q4")) == 1 and len(names) == 2, names   # + the preparation
        for (blocks, _w), cb, c, n in zip(made, c_bufs, c0, ns):
            got = gpu.download(cb, np.float32, (m, n))
            want = oracle_matmul(orc, dtype, layout, a, blocks, n, alpha=alpha, beta=beta, c=c)
            assert norm_err(got, want) < TOL and rms_err(got, want) < RMS_TOL, (n, alpha)
            cb.free()
    a_buf.free()
    for _b, w in made:
        w.free()


# Sibling weights over one activation (q/k/v, gate/up) with more than eight rows: one launch of the exact GEMM whose
# column tiles are dealt out to the weights in order. Column counts that do not fill a tile, one to four weights,
# row counts around the tile heights, alpha/beta on pre-filled outputs - each output against the oracle.
@pytest.mark.parametrize("dtype,layout", CASES)
@pytest.mark.parametrize("m,ns,k", [(37, (200, 64, 70), 256), (128, (2048, 256, 256), 2048), (9, (130,), 544), (300, (520, 1000, 8, 129), 1056)])
def test_sibling_weights_share_a_gemm_launch(gpu, orc, dtype, layout, m, ns, k):
    say("sibling gemm", dtype, layout, m, ns, k)
    made = [make_weight(gpu, orc, dtype, layout, n, k, seed=n + 7 * i, std=0.1) for i, n in enumerate(ns)]
    rng = np.random.default_rng(m)
    a = rng.standard_normal((m, k)).astype(np.float32)
    c0 = [rng.standard_normal((m, n)).astype(np.float32) for n in ns]
    a_buf = gpu.upload(a)
    for alpha, beta in ((1.0, 0.0), (0.5, -2.0)):
        c_bufs = [gpu.upload(c) for c in c0]
        gpu.profile_start()
        gpu.step_matmul_batch([w for _b, w in made], a_buf, m, c_bufs, alpha=alpha, beta=beta)
        launches = [nm for nm, _ms in gpu.profile_stop() if nm.startswith("gemm_i8")]
        assert len(launches) == 1
        for (blocks, _w), cb, c, n in zip(made, c_bufs, c0, ns):
            got = gpu.download(cb, np.float32, (m, n))
            want = oracle_matmul(orc, dtype, layout, a, blocks, n, alpha=alpha, beta=beta, c=c)
            assert norm_err(got, want) < TOL and rms_err(got, want) < RMS_TOL, (n, alpha)
            cb.free()
    a_buf.free()
    for _b, w in made:
        w.free()


@pytest.mark.parametrize("dtype,layout", CASES)
def test_exact_path_rows_above_eight(gpu, orc, dtype, layout):
    say("exact gemm", dtype, layout)
    m, n, k = 37, 200, 256
    blocks, w = make_weight(gpu, orc, dtype, layout, n, k, seed=77, std=0.1)
    a = np.random.default_rng(5).standard_normal((m, k)).astype(np.float32)
    gpu.set_gemm_mode(be.GEMM_EXACT_I8)
    got = gpu.matmul(w, a)
    want = oracle_matmul(orc, dtype, layout, a, blocks, n)
    assert norm_err(got, want) < TOL and rms_err(got, want) < RMS_TOL
    w.free()


# Shapes that exercise every workgroup shape of the LDS-staged exact kernel and its edges: K that is not a multiple
# of the 4- or 8-block K step (the blocks past the end must contribute nothing), N that is not a multiple of the
# 64/128-column tile, row counts around the 16/32/64/128-row tiles, alpha/beta on a pre-filled C.
@pytest.mark.parametrize("dtype,layout", CASES)
@pytest.mark.parametrize("m,n,k", [(17, 33, 32), (40, 130, 96), (130, 70, 288), (65, 1100, 1056), (300, 520, 800),
                                   (128, 2048, 2048), (24, 8192, 2048), (1100, 2100, 544)])
def test_exact_gemm_shapes_and_edges(gpu, orc, dtype, layout, m, n, k):
    say("exact gemm edges", dtype, layout, m, n, k)
    blocks, w = make_weight(gpu, orc, dtype, layout, n, k, seed=m + n + k, std=0.05)
    rng = np.random.default_rng(m * 7 + k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    c0 = rng.standard_normal((m, n)).astype(np.float32)
    gpu.set_gemm_mode(be.GEMM_EXACT_I8)
    got = gpu.matmul(w, a)
    assert gpu.last_kernel() == ("gemm_i8_q8" if dtype == be.Q8_0 else "gemm_i8_q4")
    want = oracle_matmul(orc, dtype, layout, a, blocks, n)
    assert norm_err(got, want) < TOL and rms_err(got, want) < RMS_TOL
    got2 = gpu.matmul(w, a, alpha=0.5, beta=-2.0, c=c0)
    want2 = 0.5 * want - 2.0 * c0
    assert rms_err(got2, want2) < RMS_TOL
    w.free()


# 2..8 activation rows (gemv_rows_kernel): row counts that fill a 2-, 4- or 8-row instance only partly, N that is
# not a multiple of the rows a wavefront works on, K of one LDS pass, K that needs most of a CU's LDS (16384 at 4 rows) and K
# long enough to run as several K-range launches (32768 at 3 rows), alpha/beta on a pre-filled C. Three shapes (5..8 rows, at
# least 16384 columns, K up to 4096) run on the 16-row tile of the LDS-staged MFMA kernel instead: ragged N, K of one and of
# many steps. Five to eight rows over a K past 4096 take the exact GEMM (its 16-row tile is far ahead there). Many weight rows
# over a K of 2048 ... 4096 take the matrix-pipe GEMV (gemv_mfma_kernel; conftest.rows_kernel states where): one wavefront per
# 16-row tile and two sharing a tile's K (14400 rows), ragged N, K of 8 / 9 / 16 stages, 3 ... 8 rows, both weight types.
@pytest.mark.parametrize("dtype,layout", CASES)
@pytest.mark.parametrize("m,n,k", [(2, 70, 96), (3, 1001, 1056), (5, 333, 2048), (8, 1030, 14336), (7, 4100, 7200), (4, 9000, 512),
                                   (5, 16390, 256), (8, 20001, 2048), (6, 16384, 4096), (4, 1030, 16384), (3, 300, 32768),
                                   (5, 70, 4128), (8, 14336, 8192), (5, 14400, 4096), (3, 65600, 2048), (8, 65539, 2304), (4, 14336, 4096), (6, 65552, 4096)])
def test_decode_gemv_two_to_eight_rows(gpu, orc, dtype, layout, m, n, k):
    say("gemv rows", dtype, layout, m, n, k)
    blocks, w = make_weight(gpu, orc, dtype, layout, n, k, seed=m * 31 + n + k, std=0.05)
    rng = np.random.default_rng(m + k)
    a = rng.standard_normal((m, k)).astype(np.float32)
    c0 = rng.standard_normal((m, n)).astype(np.float32)
    got = gpu.matmul(w, a)
    assert gpu.last_kernel() == rows_kernel(dtype == be.Q8_0, m, n, k)
    want = oracle_matmul(orc, dtype, layout, a, blocks, n)
    assert norm_err(got, want) < TOL and rms_err(got, want) < RMS_TOL
    got2 = gpu.matmul(w, a, alpha=-1.5, beta=0.25, c=c0)
    assert rms_err(got2, -1.5 * want + 0.25 * c0) < RMS_TOL
    w.free()


def test_linearity_in_alpha_and_row_independence(gpu, orc):
    # size-independent properties: rows of A never interact (the one-row and the several-row kernels give a row
    # the same int8 codes and block dots; only the order of the f32 additions over lanes may differ); alpha
    # scales exactly by powers of two
    blocks, w = make_weight(gpu, orc, be.Q4_0, be.KMAJOR_KN, 512, 1024, seed=3)
    a = np.random.default_rng(4).standard_normal((8, 1024)).astype(np.float32)
    full = gpu.matmul(w, a)
    scale = float(np.abs(full).max())
    for r in (0, 3, 7):
        assert float(np.abs(gpu.matmul(w, a[r:r + 1])[0] - full[r]).max()) <= 2e-6 * scale
    for rows in ((0, 1), (2, 3, 4, 5), (1, 7)):                          # 2- and 4-row launches against the 8-row one
        part = gpu.matmul(w, a[list(rows)])
        assert float(np.abs(part - full[list(rows)]).max()) <= 2e-6 * scale
    assert np.array_equal(gpu.matmul(w, a, alpha=4.0), 4.0 * full)
    w.free()


def test_matmul_argument_errors(gpu, orc):
    blocks, w4 = make_weight(gpu, orc, be.Q4_0, be.KMAJOR_KN, 8, 64, seed=1)
    a = gpu.upload(np.zeros((1, 64), np.float32))
    c = gpu.alloc(64)
    lib, ctx = gpu._lib, gpu._ctx
    assert lib.aionhip_step_matmul_nt(ctx, w4.ptr, 1, a.handle, 0, c.handle, 0, 1.0, 0.0) == hip.INVALID_ARGUMENT
    assert lib.aionhip_step_matmul(ctx, w4.ptr, 1, a.handle, 32, c.handle, 0, 1.0, 0.0) == hip.INVALID_ARGUMENT  # lda < k
    assert lib.aionhip_step_matmul(ctx, w4.ptr, 1, 0, 0, c.handle, 0, 1.0, 0.0) == hip.INVALID_ARGUMENT
    with pytest.raises(be.AionHipError) as e:
        gpu.upload_weight(be.Q4_0, be.ROWS_NK, 8, 64, blocks)           # aion has no q4 [N,K] operand
    assert e.value.status == hip.UNSUPPORTED
    with pytest.raises(be.AionHipError) as e:
        gpu.upload_weight(be.Q8_0, be.ROWS_NK, 8, 48, np.zeros(8 * 2 * 34, np.uint8))
    assert e.value.status == hip.INVALID_ARGUMENT
    assert lib.aionhip_step_matmul(ctx, w4.ptr, 0, a.handle, 0, c.handle, 0, 1.0, 0.0) == hip.OK   # m == 0 is a no-op
    a.free(); c.free(); w4.free()


@pytest.mark.parametrize("dtype,layout", CASES)
def test_single_row_fused_kernel_equals_prepared_path(gpu, orc, dtype, layout):
    # m == 1 builds the int8 activation inside the GEMV; a 2-row call goes through prepare_act + gemv.
    # Same codes, same scales, same per-lane order: the shared row must agree bit for bit.
    for n, k in [(67, 2080), (2048, 2048), (300, 4096)]:
        blocks, w = make_weight(gpu, orc, dtype, layout, n, k, seed=n + k)
        a = np.random.default_rng(n).standard_normal((2, k)).astype(np.float32)
        one = gpu.matmul(w, a[:1])
        assert gpu.last_kernel().endswith("_fused")
        two = gpu.matmul(w, a)
        assert not gpu.last_kernel().endswith("_fused")
        assert np.array_equal(one[0], two[0])
        w.free()


# Two rows and more on the exact kernels take the norm and the int8 preparation as one launch: rows of up to 2048 columns
# (everything requested before the reduction) and longer ones (two passes), column counts that leave the last 256-thread pass
# partly empty, with and without the norm's beta, 2..8 rows (GEMV) and more (GEMM) - the bits of the norm step followed by the
# matmul step, and one launch fewer.
@pytest.mark.parametrize("k", [96, 1056, 2048, 2080, 4096, 8224])
@pytest.mark.parametrize("rows,with_beta", [(2, False), (5, True), (9, True), (70, False)])
def test_rmsnorm_and_preparation_in_one_launch_give_the_bits_of_the_two_steps(gpu, orc, k, rows, with_beta):
    say("rmsnorm + prepare", k, rows, with_beta)
    rng = np.random.default_rng(k + rows)
    n = 72
    _b, w = make_weight(gpu, orc, be.Q4_0, be.KMAJOR_KN, n, k, seed=k)
    x = (rng.standard_normal((rows, k)) * (1 + rng.random((rows, 1)) * 5)).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    beta = (0.1 * rng.standard_normal(k)).astype(np.float32)
    xb, gb, bb = gpu.upload(x), gpu.upload(gamma), (gpu.upload(beta) if with_beta else None)
    c1, c2, hb = gpu.alloc(rows * n * 4), gpu.alloc(rows * n * 4), gpu.alloc(rows * k * 4)
    gpu.set_gemm_mode(be.GEMM_EXACT_I8)
    gpu.profile_start()
    gpu.step_rmsnorm_matmul([w], xb, gb, rows, [c1], 1e-6, beta_norm=bb)
    names = [nm for nm, _ in gpu.profile_stop()]
    assert names[0] == "prepare_rmsnorm" and "prepare_act" not in names, names
    gpu.step_rmsnorm(hb, xb, gb, rows, k, 1e-6, beta=bb)
    gpu.step_matmul(w, hb, rows, c2)
    assert np.array_equal(gpu.download(c1, np.float32, (rows, n)), gpu.download(c2, np.float32, (rows, n)))
    for t in (xb, gb, c1, c2, hb) + ((bb,) if bb is not None else ()):
        t.free()
    w.free()


@pytest.mark.parametrize("dtype,layout", CASES)
@pytest.mark.parametrize("rows", [1, 3, 6, 40])
def test_rmsnorm_matmul_and_gate_matmul_match_the_separate_steps(gpu, orc, dtype, layout, rows):
    say("fused steps", dtype, layout, rows)
    rng = np.random.default_rng(rows + dtype)
    k, n1, n2 = 2048, 512, 96
    b1, w1 = make_weight(gpu, orc, dtype, layout, n1, k, seed=1)
    b2, w2 = make_weight(gpu, orc, dtype, layout, n2, k, seed=2)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    xb, gb = gpu.upload(x), gpu.upload(gamma)
    c1, c2 = gpu.alloc(rows * n1 * 4), gpu.alloc(rows * n2 * 4)
    gpu.step_rmsnorm_matmul([w1, w2], xb, gb, rows, [c1, c2], 1e-6)
    if rows == 1:
        assert gpu.last_kernel().endswith("_rmsnorm")
    got1, got2 = gpu.download(c1, np.float32, (rows, n1)), gpu.download(c2, np.float32, (rows, n2))
    if rows > 1:
        # several rows: the step is the norm step followed by the matmul step on the normalised rows, so the same bits come out
        hb, d1, d2 = gpu.alloc(rows * k * 4), gpu.alloc(rows * n1 * 4), gpu.alloc(rows * n2 * 4)
        gpu.step_rmsnorm(hb, xb, gb, rows, k, 1e-6)
        gpu.step_matmul_batch([w1, w2], hb, rows, [d1, d2])
        assert np.array_equal(gpu.download(d1, np.float32, (rows, n1)), got1)
        assert np.array_equal(gpu.download(d2, np.float32, (rows, n2)), got2)
        for t in (hb, d1, d2):
            t.free()
    h = orc.rmsnorm(x, gamma, 1e-6)
    want1, want2 = oracle_matmul(orc, dtype, layout, h, b1, n1), oracle_matmul(orc, dtype, layout, h, b2, n2)
    # the norm's sum of squares is reduced in a different order than on the CPU: an activation on a
    # rounding boundary may take the neighbouring int8 code, worth up to ~1e-3 of rms per flipped code
    assert rms_err(got1, want1) < 3e-3 and rms_err(got2, want2) < 3e-3
    # gate: act = gelu(gate) * up, K = ffn
    gate = (rng.standard_normal((rows, k)) * 2).astype(np.float32)
    up = rng.standard_normal((rows, k)).astype(np.float32)
    gtb, upb = gpu.upload(gate), gpu.upload(up)
    res0 = rng.standard_normal((rows, n1)).astype(np.float32)
    cres = gpu.upload(res0)
    gpu.step_gate_matmul(w1, gtb, upb, rows, cres, beta=1.0)          # accumulates into C: a fused residual add
    if rows == 1:
        assert gpu.last_kernel().endswith("_gate")
    act = orc.gate_gelu(gate, up).reshape(rows, k)
    want = oracle_matmul(orc, dtype, layout, act, b1, n1, beta=1.0, c=res0)
    assert rms_err(gpu.download(cres, np.float32, (rows, n1)), want) < 3e-3
    # a long reduction axis (K = 8192) takes the gate + preparation launch, then the GEMV
    b3, w3 = make_weight(gpu, orc, dtype, layout, 160, 8192, seed=3)
    gate8 = (rng.standard_normal((rows, 8192)) * 2).astype(np.float32)
    up8 = rng.standard_normal((rows, 8192)).astype(np.float32)
    g8, u8, c8 = gpu.upload(gate8), gpu.upload(up8), gpu.alloc(rows * 160 * 4)
    gpu.step_gate_matmul(w3, g8, u8, rows, c8)
    want8 = oracle_matmul(orc, dtype, layout, orc.gate_gelu(gate8, up8).reshape(rows, 8192), b3, 160)
    assert rms_err(gpu.download(c8, np.float32, (rows, 160)), want8) < 3e-3
    for t in (xb, gb, c1, c2, gtb, upb, cres, g8, u8, c8):
        t.free()
    w1.free(); w2.free(); w3.free()


# K between 4096 and 8192 with 16384 or more outputs in the call: one row keeps the fused kernels (eight activation chunks
# per thread), with the RMSNorm and the gate prologues as well; the outputs of two sibling weights count together.
@pytest.mark.parametrize("dtype,layout", CASES)
def test_fused_prologues_at_k_up_to_8192_with_many_outputs(gpu, orc, dtype, layout):
    rng = np.random.default_rng(11 + dtype)
    k, n1, n2 = 6176, 9000, 7400
    b1, w1 = make_weight(gpu, orc, dtype, layout, n1, k, seed=1)
    b2, w2 = make_weight(gpu, orc, dtype, layout, n2, k, seed=2)
    x = rng.standard_normal((1, k)).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    xb, gb = gpu.upload(x), gpu.upload(gamma)
    c1, c2 = gpu.alloc(n1 * 4), gpu.alloc(n2 * 4)
    gpu.step_rmsnorm_matmul([w1, w2], xb, gb, 1, [c1, c2], 1e-6)
    assert gpu.last_kernel().endswith("_rmsnorm")
    h = orc.rmsnorm(x, gamma, 1e-6)
    assert rms_err(gpu.download(c1, np.float32, (1, n1)), oracle_matmul(orc, dtype, layout, h, b1, n1)) < 3e-3
    assert rms_err(gpu.download(c2, np.float32, (1, n2)), oracle_matmul(orc, dtype, layout, h, b2, n2)) < 3e-3
    gpu.step_rmsnorm_matmul([w1], xb, gb, 1, [c1], 1e-6)           # 9000 outputs alone: norm kernel, then the K slices
    assert not gpu.last_kernel().endswith("_rmsnorm")
    assert rms_err(gpu.download(c1, np.float32, (1, n1)), oracle_matmul(orc, dtype, layout, h, b1, n1)) < 3e-3
    w1.free(); w2.free()
    n3 = 16384
    b3, w3 = make_weight(gpu, orc, dtype, layout, n3, 8192, seed=3)
    gate = (rng.standard_normal((1, 8192)) * 2).astype(np.float32)
    up = rng.standard_normal((1, 8192)).astype(np.float32)
    res0 = rng.standard_normal((1, n3)).astype(np.float32)
    g8, u8, c3 = gpu.upload(gate), gpu.upload(up), gpu.upload(res0)
    gpu.step_gate_matmul(w3, g8, u8, 1, c3, beta=1.0)
    assert gpu.last_kernel().endswith("_gate")
    want = oracle_matmul(orc, dtype, layout, orc.gate_gelu(gate, up).reshape(1, 8192), b3, n3, beta=1.0, c=res0)
    assert rms_err(gpu.download(c3, np.float32, (1, n3)), want) < 3e-3
    # sibling weights in one call stay on the fused kernel whatever their size (there is no K-slice form for them)
    b4, w4 = make_weight(gpu, orc, dtype, layout, 300, k, seed=4)
    b5, w5 = make_weight(gpu, orc, dtype, layout, 72, k, seed=5)
    c4, c5 = gpu.alloc(300 * 4), gpu.alloc(72 * 4)
    gpu.step_matmul_batch([w4, w5], xb, 1, [c4, c5])
    assert gpu.last_kernel().endswith("_fused")
    assert rms_err(gpu.download(c4, np.float32, (1, 300)), oracle_matmul(orc, dtype, layout, x, b4, 300)) < RMS_TOL
    assert rms_err(gpu.download(c5, np.float32, (1, 72)), oracle_matmul(orc, dtype, layout, x, b5, 72)) < RMS_TOL
    for t in (xb, gb, c1, c2, g8, u8, c3, c4, c5):
        t.free()
    w3.free(); w4.free(); w5.free()


# MatMulNT with an f32 B [N,K] (runtime/executable.zig:211-223; cpu/kernels/matmul_nt.zig:40-126): nothing is quantized.
# Exact inputs (small integers: every partial sum exact in f32, so every summation order gives the same bits) must come out
# bit-equal to the oracle; random inputs are held to the float64 product within twice the oracle's own distance from it
# (the device sums the same terms in another order). Shapes: one row and many, K that is not a multiple of 4 (scalar loads),
# K below a wavefront, a vocabulary-sized N, strides and alpha / beta; then what an f32 weight is refused for.
@pytest.mark.parametrize("m,n,k", [(1, 7, 1), (1, 1000, 4096), (3, 129, 100), (8, 64, 2048), (21, 300, 515), (5, 40000, 512), (2, 5, 4099)])
def test_matmul_nt_with_an_f32_weight(gpu, orc, m, n, k):
    say("matmul_nt f32", m, n, k)
    rng = np.random.default_rng(m * 7 + n + k)
    wi = rng.integers(-8, 9, (n, k)).astype(np.float32)
    ai = rng.integers(-8, 9, (m, k)).astype(np.float32)
    w = gpu.upload_weight(be.F32, be.ROWS_NK, n, k, wi)
    assert w.packed_bytes == n * k * 4 and np.array_equal(w.download().view(np.float32).reshape(n, k), wi)
    got = gpu.matmul(w, ai)
    assert gpu.last_kernel() == "matmul_nt_f32"
    assert np.array_equal(got, orc.matmul_nt_f32(ai, wi)) and np.array_equal(got, (ai.astype(np.int64) @ wi.astype(np.int64).T).astype(np.float32))
    c0 = rng.integers(-4, 5, (m, n)).astype(np.float32)
    assert np.array_equal(gpu.matmul(w, ai, alpha=2.0, beta=-0.5, c=c0), orc.matmul_nt_f32(ai, wi, alpha=2.0, beta=-0.5, c=c0))
    w.free()
    wf = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    af = rng.standard_normal((m, k)).astype(np.float32)
    w = gpu.upload_weight(be.F32, be.ROWS_NK, n, k, wf)
    got = gpu.matmul(w, af)
    ref64 = af.astype(np.float64) @ wf.astype(np.float64).T
    want = orc.matmul_nt_f32(af, wf)
    rms = float(np.sqrt((ref64 ** 2).mean()))
    own = float(np.abs(want - ref64).max())
    err = float(np.abs(got - ref64).max())
    say("   max|err| vs f64: device", err / rms, "oracle", own / rms)
    assert err <= 2 * own + 1e-7 * rms
    assert float(np.abs(got - want).max()) <= 1e-5 * rms
    w.free()


def test_an_f32_weight_is_a_matmul_nt_operand_only(gpu):
    n, k = 64, 64
    wf = np.ones((n, k), np.float32)
    with pytest.raises(be.AionHipError) as e:
        gpu.upload_weight(be.F32, be.KMAJOR_KN, n, k, wf)
    assert e.value.status == hip.UNSUPPORTED
    w = gpu.upload_weight(be.F32, be.ROWS_NK, n, k, wf)
    x, g, c = gpu.upload(np.ones((1, k), np.float32)), gpu.upload(np.ones(k, np.float32)), gpu.zeros(n * 4)
    with pytest.raises(be.AionHipError) as e:
        gpu.step_rmsnorm_matmul([w], x, g, 1, [c], 1e-6)
    assert e.value.status == hip.UNSUPPORTED
    with pytest.raises(be.AionHipError) as e:
        gpu.step_matmul_batch([w, w], x, 1, [c, c])
    assert e.value.status == hip.UNSUPPORTED
    gpu.step_matmul(w, x, 1, c)                      # the plain step runs
    assert np.array_equal(gpu.download(c, np.float32, (n,)), np.full(n, k, np.float32))
    # a strided A and C: lda / ldc in elements
    a2 = np.arange(2 * 80, dtype=np.float32).reshape(2, 80) % 7
    ab, cb = gpu.upload(a2), gpu.zeros(2 * 100 * 4)
    gpu.step_matmul(w, ab, 2, cb, lda=80, ldc=100)
    out = gpu.download(cb, np.float32, (2, 100))
    assert np.array_equal(out[:, :n], np.repeat(a2[:, :k].sum(axis=1, keepdims=True), n, axis=1)) and not out[:, n:].any()
    for t in (x, g, c, ab, cb):
        t.free()
    w.free()
