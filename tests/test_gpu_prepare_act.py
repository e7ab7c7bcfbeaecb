"""The int8 activation preparation of every kernel that does one, bit for bit against the oracle's prepare_a
(aion cpu/kernels/matmul_q_i8.zig:187-203, 227-264), read out through the C ABI.

A block-form identity weight (act_cases.py) makes C[n] = f32(code[n % K]) * a_scale[block], so the matmul's output IS the
prepared activation; the q4 identity also needs the per-block code sums to be right. The rows hold exact rounding ties,
zero blocks, an amax on a negative element, a denormal amax, and values that tell 127 / amax from 1 / (amax / 127).
Bar: bit-exact (np.array_equal on f32).
"""
import sys

import numpy as np
import pytest

import act_cases as ac
from aion_amd import backend as be

pytestmark = pytest.mark.gpu

WEIGHTS = [("q8_rows", be.Q8_0, be.ROWS_NK, ac.identity_q8_rows), ("q8_kmajor", be.Q8_0, be.KMAJOR_KN, ac.identity_q8_kmajor),
           ("q4_kmajor", be.Q4_0, be.KMAJOR_KN, ac.identity_q4_kmajor)]


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def identity(gpu, kind, n, k):
    _name, dtype, layout, make = next(w for w in WEIGHTS if w[0] == kind)
    return gpu.upload_weight(dtype, layout, n, k, make(n, k))


# (rows, n, k, kernel that must have run): the one-row kernel with the preparation inside (256- and 1024-thread forms share
# the code; K = 4096 fills all four chunks per thread), the K-split one-row kernel for K > 4096 (each workgroup prepares its
# slice), the 2..8-row kernel behind the separate preparation launch, the 16-row tile of the exact GEMM for 5..8 rows against a wide weight, the exact GEMM.
PRODUCERS = [(1, 512, 512, "gemv_%s_fused"), (1, 4096, 4096, "gemv_%s_fused"), (1, 4160, 4160, "gemv_%s_ksplit"), (1, 600, 14336, "gemv_%s_ksplit"),
             (2, 512, 512, "gemv_%s"), (4, 1056, 1056, "gemv_%s"), (8, 512, 512, "gemv_%s"), (3, 96, 8192, "gemv_%s"),
             (6, 16384, 512, "gemv_%s"), (20, 512, 512, "gemm_i8_%s"), (130, 300, 1056, "gemm_i8_%s")]


@pytest.mark.parametrize("kind", [w[0] for w in WEIGHTS])
@pytest.mark.parametrize("m,n,k,kernel", PRODUCERS)
def test_prepared_activation_read_out_bit_exact(gpu, orc, kind, m, n, k, kernel):
    say("prepare_act readout", kind, m, n, k)
    w = identity(gpu, kind, n, k)
    a = ac.rows(m, k, seed=m * 1000 + k)
    gpu.set_gemm_mode(be.GEMM_EXACT_I8)
    got = gpu.matmul(w, a)
    assert gpu.last_kernel() == kernel % kind[:2]
    want = ac.expected_readout(orc, a, n)
    assert got.dtype == want.dtype == np.float32
    bad = np.argwhere(got.view(np.uint32) != want.view(np.uint32))
    assert bad.size == 0, (bad[:5], got[tuple(bad[0])], want[tuple(bad[0])])
    w.free()


@pytest.mark.parametrize("kind", [w[0] for w in WEIGHTS])
@pytest.mark.parametrize("rows,k", [(1, 512), (1, 4096), (1, 4160), (3, 512)])
def test_norm_and_gate_prologues_prepare_the_same_codes(gpu, orc, kind, rows, k):
    # RMSNorm with gamma = 0 and beta = a yields a exactly ((x * inv_rms) * 0 + a); gelu_tanh(16) = 16 exactly (the tanh
    # saturates to 1), so gate = 16, up = a / 16 yields a exactly: both fused prologues (and the separate gate + preparation
    # launch for several rows or long K) must then read out the same bits as the plain preparation.
    say("prologue readout", kind, rows, k)
    w = identity(gpu, kind, k, k)
    a = ac.rows(rows, k, seed=rows + k, denormal=False)           # a / 16 below must stay exact
    want = ac.expected_readout(orc, a, k)
    x = gpu.upload(np.random.default_rng(k).standard_normal((rows, k)).astype(np.float32))
    gamma, c = gpu.zeros(k * 4), gpu.alloc(rows * k * 4)
    if rows == 1:       # the norm's beta is one vector for all rows
        beta = gpu.upload(a[0])
        gpu.step_rmsnorm_matmul([w], x, gamma, 1, [c], 1e-6, beta_norm=beta)
        if k <= 4096:
            assert gpu.last_kernel().endswith("_rmsnorm")
        got = gpu.download(c, np.float32, (1, k))
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        beta.free()
    a16 = (a / np.float32(16)).astype(np.float32)
    assert np.array_equal(a16 * np.float32(16), a)
    gate, up = gpu.upload(np.full((rows, k), 16.0, np.float32)), gpu.upload(a16)
    gpu.step_gate_matmul(w, gate, up, rows, c)
    if rows == 1 and k <= 4096:
        assert gpu.last_kernel().endswith("_gate")
    got = gpu.download(c, np.float32, (rows, k))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    for t in (x, gamma, c, gate, up):
        t.free()
    w.free()


def test_geglu_epilogue_prepares_the_same_codes(gpu, orc):
    # aionhip_step_rmsnorm_geglu_matmul quantizes h = gelu(g) * u inside the gate/up kernel. Make h exact: the norm yields its
    # beta (gamma = 0) = one block with codes (127, 1, 0, ...) at scale 1; gate row j has code 1 at position 1, scale 16
    # -> g_j = 16 = gelu(16); up row j has code c_j at position 1, scale s_j -> u_j = c_j * s_j; h_j = 16 * c_j * s_j.
    # The down weight is the identity, so the output is f32(code(h)_j) * scale(h)_block.
    hidden = 64
    h = np.concatenate([np.array([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -63.5, 62.5, -61.5, 0.0, 3.5, 4.5, -4.5, 5.5,
                                  6.5, -7.5, 8.5, 9.5, 10.5, -11.5, 12.5, 13.5, 0.0, 0.0, 21.5, -22.5, 33.5, 44.5, -55.5, 60.5], np.float32),
                        np.zeros(32, np.float32),
                        np.array(ac.HALF_BLOCK, np.float32)])
    F = h.size
    # factor h_j / 16 = c_j * s_j with |c_j| <= 127 an integer and s_j a power of two
    u = h / np.float32(16)
    c_up, s_up = np.zeros(F, np.int64), np.ones(F, np.float32)
    for j, v in enumerate(u):
        if v != 0:
            s = np.float32(1.0)
            while float(v / s) != round(float(v / s)):
                s = np.float32(s / 2)
            while abs(v / s) > 127:
                s = np.float32(s * 2)
            assert float(v / s) == round(float(v / s)) and abs(v / s) <= 127, (j, v)
            c_up[j], s_up[j] = int(v / s), s
    kb = hidden // 32

    def rows_weight(codes_at_1, scales):
        b = np.zeros((F, kb, 34), np.uint8)
        b[:, :, 0:2] = np.array([1.0], np.float16).view(np.uint8)
        b[:, 0, 0:2] = scales.astype(np.float16).view(np.uint8).reshape(F, 2)
        b[:, 0, 2 + 1] = codes_at_1.astype(np.int8).view(np.uint8)
        return gpu.upload_weight(be.Q8_0, be.ROWS_NK, F, hidden, b.reshape(-1))

    wg = rows_weight(np.ones(F, np.int64), np.full(F, 16.0, np.float32))
    wu = rows_weight(c_up, s_up)
    wd = gpu.upload_weight(be.Q8_0, be.ROWS_NK, F, F, ac.identity_q8_rows(F, F))
    beta = np.zeros(hidden, np.float32)
    beta[0], beta[1] = 127.0, 1.0
    x = gpu.upload(np.random.default_rng(1).standard_normal((1, hidden)).astype(np.float32))
    gamma, bb, c = gpu.zeros(hidden * 4), gpu.upload(beta), gpu.alloc(F * 4)
    gpu.step_rmsnorm_geglu_matmul(wg, wu, wd, x, gamma, 1e-6, c, beta_norm=bb)
    got = gpu.download(c, np.float32, (1, F))
    want = ac.expected_readout(orc, h.reshape(1, F), F)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (got, want)
    # and the separate steps give the same read-out
    g_buf, u_buf = gpu.alloc(F * 4), gpu.alloc(F * 4)
    gpu.step_rmsnorm_matmul([wg, wu], x, gamma, 1, [g_buf, u_buf], 1e-6, beta_norm=bb)
    assert np.array_equal(gpu.download(g_buf, np.float32, (F,)), np.full(F, 16.0, np.float32))
    assert np.array_equal(gpu.download(u_buf, np.float32, (F,)), u)
    for t in (x, gamma, bb, c, g_buf, u_buf):
        t.free()
    for w in (wg, wu, wd):
        w.free()
