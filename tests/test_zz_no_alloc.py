"""aionhip_step_matmul_static - the matmul step for callers that cannot allocate - against aionhip_step_matmul /
aionhip_step_matmul_nt on the same operands, through the C ABI. Where both run the same kernel the same way the bar is bit
equality. Two cases differ in the order of their f32 additions only - the same int8 codes and block dots - and are held to
max|diff| <= 1e-5 * rms like every exact-integer-dot kernel against the oracle: one row against K > 4096 runs the K-split
kernel in the allocating entry point (it keeps a growable buffer) and the separate preparation + one-row kernel in the
static one; and the exact GEMM cuts a long K into slices across workgroups when its grid is sparse, through a buffer of
partial sums that the static entry point may not take.

Every call on a GPU shares one static device array that keeps the last call's contents: the calls come in pairs, the second
with a smaller input than the first (fewer rows, shorter K), so stale bytes of the first call lie right behind the second
call's planes.
"""
import sys

import numpy as np
import pytest

from aion_amd import backend as be
from aion_amd import hip

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def make(gpu, dtype, layout, n, k, seed):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((n, k) if layout == be.ROWS_NK else (k, n)) * 0.05).astype(np.float32)
    return gpu.upload_weight(dtype, layout, n, k, be.quantize_blocks(dtype, w, 1 if layout == be.ROWS_NK else 0))


def both(gpu, w, a, alpha=1.0, beta=0.0, c0=None):
    """-> (existing entry point's C, static entry point's C, whether both ran the same kernel)"""
    m = a.shape[0]
    a_buf = gpu.upload(a)
    outs, kernels = [], []
    for fn in (gpu.step_matmul, gpu.step_matmul_static):
        c_buf = gpu.upload(c0) if c0 is not None else gpu.zeros(m * w.n * 4)
        fn(w, a_buf, m, c_buf, alpha=alpha, beta=beta)
        kernels.append(gpu.last_kernel())
        outs.append(gpu.download(c_buf, np.float32, (m, w.n)))
        c_buf.free()
    a_buf.free()
    return outs[0], outs[1], kernels[0] == kernels[1] and not kernels[0].startswith("gemm_i8")


def same(want, got, same_kernel):
    if same_kernel:
        return np.array_equal(want.view(np.uint32), got.view(np.uint32))
    return float(np.abs(got - want).max()) <= 1e-5 * float(np.sqrt((want.astype(np.float64) ** 2).mean()))


@pytest.mark.parametrize("dtype,layout", [(be.Q4_0, be.KMAJOR_KN), (be.Q8_0, be.ROWS_NK), (be.Q8_0, be.KMAJOR_KN)])
def test_static_entry_point_equals_the_allocating_one_on_two_calls_in_a_row(gpu, orc, dtype, layout):
    say("no-alloc entry", dtype, layout)
    gpu.set_gemm_mode(be.GEMM_EXACT_I8)
    rng = np.random.default_rng(dtype * 7 + layout)
    # (first call, then a smaller one): 2..8-row kernel, one row past K = 4096 (separate preparation), exact GEMM
    for (m1, n1, k1), (m2, n2, k2) in [((8, 3000, 2048), (3, 515, 1056)), ((1, 2050, 8224), (1, 300, 4128)),
                                       ((4, 20000, 512), (2, 70, 96)), ((100, 520, 2048), (17, 33, 160)),
                                       ((7, 16390, 256), (5, 16384, 128))]:
        for (m, n, k) in ((m1, n1, k1), (m2, n2, k2)):
            w = make(gpu, dtype, layout, n, k, seed=n + k)
            a = rng.standard_normal((m, k)).astype(np.float32)
            want, got, same_kernel = both(gpu, w, a)
            assert same_kernel == (not (m == 1 and k > 4096) and m <= 8)
            assert same(want, got, same_kernel), (m, n, k)
            ref = orc.matmul_nt_q8(a, w.download(), n, threads=8) if layout == be.ROWS_NK else orc.matmul_q_packed(dtype, a, w.download(), n, threads=8)
            assert float(np.abs(got - ref).max()) <= 1e-5 * float(np.sqrt((ref.astype(np.float64) ** 2).mean()))
            c0 = rng.standard_normal((m, n)).astype(np.float32)
            want, got, same_kernel = both(gpu, w, a, alpha=0.5, beta=-2.0, c0=c0)
            assert same(want, got, same_kernel), (m, n, k, "alpha/beta")
            w.free()


def test_static_entry_point_rejects_what_does_not_fit_or_would_allocate(gpu):
    lib, ctx = gpu._lib, gpu._ctx
    k = 32768
    w = make(gpu, be.Q8_0, be.ROWS_NK, 8, k, seed=1)
    m = 40                                          # 40 * 32768 bytes of codes alone exceed the 1 MiB array
    a, c = gpu.zeros(m * k * 4), gpu.zeros(m * 8 * 4)
    assert lib.aionhip_step_matmul_static(ctx, w.ptr, m, a.handle, 0, c.handle, 0, 1.0, 0.0) == hip.INVALID_ARGUMENT
    assert b"static scratch holds" in lib.aionhip_last_error(ctx)
    assert lib.aionhip_step_matmul_static(ctx, w.ptr, 8, a.handle, 0, c.handle, 0, 1.0, 0.0) == hip.OK      # 8 rows fit
    gpu.set_gemm_mode(be.GEMM_BF16_MFMA_ALWAYS)
    assert lib.aionhip_step_matmul_static(ctx, w.ptr, 9, a.handle, 0, c.handle, 0, 1.0, 0.0) == hip.UNSUPPORTED
    gpu.set_gemm_mode(be.GEMM_EXACT_I8)
    gpu.profile_start()
    assert lib.aionhip_step_matmul_static(ctx, w.ptr, 2, a.handle, 0, c.handle, 0, 1.0, 0.0) == hip.UNSUPPORTED
    gpu.profile_stop()
    assert lib.aionhip_step_matmul_static(ctx, w.ptr, 0, a.handle, 0, c.handle, 0, 1.0, 0.0) == hip.OK      # m == 0: no-op
    assert lib.aionhip_step_matmul_static(ctx, w.ptr, 1, 0, 0, c.handle, 0, 1.0, 0.0) == hip.INVALID_ARGUMENT
    gpu.sync()
    a.free(); c.free(); w.free()


def test_static_entry_point_inside_a_recorded_program(gpu, orc):
    # the caller this entry point exists for: a step recorded into a HIP graph, where nothing may allocate - without any
    # eager warm-up call to size a scratch buffer first
    n, k, m = 1030, 8224, 3
    w = make(gpu, be.Q4_0, be.KMAJOR_KN, n, k, seed=5)
    a = np.random.default_rng(6).standard_normal((m, k)).astype(np.float32)
    a_buf, c_buf = gpu.upload(a), gpu.zeros(m * n * 4)
    gpu.program_begin()
    try:
        gpu.step_matmul_static(w, a_buf, m, c_buf)
    finally:
        prog = gpu.program_end()
    ref = orc.matmul_q_packed(be.Q4_0, a, w.download(), n, threads=8)
    rms = float(np.sqrt((ref.astype(np.float64) ** 2).mean()))
    for _ in range(3):
        gpu._check(gpu._lib.aionhip_memset(gpu._ctx, c_buf.handle, 0, 0, m * n * 4))
        gpu.program_execute(prog)
        got = gpu.download(c_buf, np.float32, (m, n))
        assert float(np.abs(got - ref).max()) <= 1e-5 * rms
    gpu.program_destroy(prog)
    a_buf.free(); c_buf.free(); w.free()


def _device_free_bytes():
    import ctypes as C
    rt = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(0), C.c_size_t(0)
    assert rt.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


# one case per route the static entry point can take: one row with the preparation inside the kernel; one row past K = 8192
# (separate preparation + one-row kernel); 2..8 rows (preparation + rows kernel); 5..8 rows against a wide short weight (the
# 16-row MFMA tile); more than 8 rows (the exact GEMM, whose K slices need a buffer and are therefore off here)
ROUTES = [("one row, fused", be.Q4_0, be.KMAJOR_KN, 1, 2100, 4096), ("one row, long K", be.Q8_0, be.ROWS_NK, 1, 520, 16416),
          ("few rows", be.Q8_0, be.KMAJOR_KN, 3, 1030, 2048), ("few rows, 16-row tile", be.Q4_0, be.KMAJOR_KN, 6, 16390, 1024),
          ("few rows, matrix pipe", be.Q4_0, be.KMAJOR_KN, 5, 14400, 2048), ("exact GEMM", be.Q4_0, be.KMAJOR_KN, 24, 520, 8192)]


def test_every_route_records_on_a_fresh_context_and_allocates_nothing(orc):
    """A context on which NO eager step ever ran (no scratch buffer has a size yet): every route of the static entry point is
    recorded into a program - stream capture rejects an allocation, so a clean recording shows the route made none - and
    replayed against the oracle; then the same calls eagerly, with the library's own counters and the device's free memory
    unchanged around them."""
    g = be.HipBackend(0)
    try:
        g.set_gemm_mode(be.GEMM_EXACT_I8)
        rng = np.random.default_rng(77)
        cases = []
        for name, dtype, layout, m, n, k in ROUTES:
            w = make(g, dtype, layout, n, k, seed=n + k + m)
            a = rng.standard_normal((m, k)).astype(np.float32)
            cases.append((name, dtype, layout, m, n, k, w, a, g.upload(a), g.zeros(m * n * 4)))
        g.sync()
        for name, dtype, layout, m, n, k, w, a, a_buf, c_buf in cases:
            say("no-alloc route", name)
            g.program_begin()
            try:
                g.step_matmul_static(w, a_buf, m, c_buf)
            finally:
                prog = g.program_end()
            ref = orc.matmul_nt_q8(a, w.download(), n, threads=8) if layout == be.ROWS_NK else orc.matmul_q_packed(dtype, a, w.download(), n, threads=8)
            rms = float(np.sqrt((ref.astype(np.float64) ** 2).mean()))
            for _ in range(2):
                g._check(g._lib.aionhip_memset(g._ctx, c_buf.handle, 0, 0, m * n * 4))
                g.program_execute(prog)
                got = g.download(c_buf, np.float32, (m, n))
                assert float(np.abs(got - ref).max()) <= 1e-5 * rms, name
            g.program_destroy(prog)
        g.sync()
        stats0, free0 = g.memory_stats(), _device_free_bytes()
        for name, dtype, layout, m, n, k, w, a, a_buf, c_buf in cases:
            g.step_matmul_static(w, a_buf, m, c_buf)
        g.sync()
        assert g.memory_stats() == stats0 and _device_free_bytes() == free0
        for case in cases:
            case[6].free(); case[8].free(); case[9].free()
    finally:
        g.close()
