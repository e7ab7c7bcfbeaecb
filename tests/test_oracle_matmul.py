"""Pins the oracle's int8-activation matmuls (CPU only).

Checks: the reference's own closed-form test inputs evaluated with its f64 formula
(matvec_q.zig:176-219, matmul_nt_q.zig:587-637), brute-force integer identities, the special
case where activation quantization is lossless (reduces to a dequantized f64 matmul), layout
invariants (K-major == NT on permuted blocks; strided == compact), alpha/beta, K chunking.
"""
import numpy as np
import pytest


def np_prepare_a(a):
    a = a.astype(np.float32)
    m, k = a.shape
    blk = a.reshape(m, k // 32, 32)
    amax = np.abs(blk).max(axis=2)
    with np.errstate(divide="ignore", invalid="ignore"):
        inv = np.where(amax == 0, np.float32(0), np.float32(127) / amax).astype(np.float32)
    prod = (blk * inv[:, :, None]).astype(np.float32).astype(np.float64)
    q = np.clip(np.sign(prod) * np.floor(np.abs(prod) + 0.5), -127, 127).astype(np.int8)
    scale = np.where(amax == 0, np.float32(0), amax / np.float32(127)).astype(np.float32)
    return q.reshape(m, k), scale


def f64_formula(aq, a_s, wq, w_s):
    """sum_kb a_s*w_s*idot in f64. aq [m,k] i8, a_s [m,kb], wq [n,k] i8, w_s [n,kb]."""
    m, k = aq.shape
    n = wq.shape[0]
    idot = np.einsum("mbt,nbt->mnb", aq.reshape(m, -1, 32).astype(np.int64), wq.reshape(n, -1, 32).astype(np.int64))
    return (idot.astype(np.float64) * a_s.astype(np.float64)[:, None, :] * w_s.astype(np.float64)[None, :, :]).sum(axis=2)


def split_q8(blocks, n, kb):
    b = blocks.reshape(n, kb, 34)
    s = b[:, :, 0:2].copy().view(np.float16).reshape(n, kb).astype(np.float32)
    q = b[:, :, 2:].copy().view(np.int8).reshape(n, kb * 32)
    return q, s


def split_q4(blocks, n, kb):
    b = blocks.reshape(n, kb, 18)
    s = b[:, :, 0:2].copy().view(np.float16).reshape(n, kb).astype(np.float32)
    nib = b[:, :, 2:]
    q = np.stack([nib & 15, nib >> 4], axis=3).reshape(n, kb * 32).astype(np.int16) - 8
    return q.astype(np.int8), s


def test_prepare_a_brute_force_and_bias_identity(orc):
    rng = np.random.default_rng(3)
    a = rng.standard_normal((5, 96)).astype(np.float32)
    a[1, 32:64] = 0.0
    a[2, 0] = 1e-30
    aq, sc, sm = orc.prepare_a(a)
    q, s = np_prepare_a(a)
    assert np.array_equal(aq, q) and np.array_equal(sc, s)
    assert np.array_equal(sm, aq.reshape(5, 3, 32).astype(np.int32).sum(axis=2))
    assert (np.abs(aq.astype(int)) <= 127).all() and (aq[1, 32:64] == 0).all() and sc[1, 1] == 0.0
    # matmul_q_i8.zig:864-889: (a+128 as u8) . b - 128*sum(b) == a . b
    b = rng.integers(-128, 128, (96,), dtype=np.int64)
    au = aq.astype(np.int64) + 128
    assert np.array_equal(au @ b - 128 * b.sum(), aq.astype(np.int64) @ b)


def test_kmajor_reference_closed_form_past_chunk(orc):
    # matvec_q.zig:176-219: m=2, n=5, k=8192+64; a[i]=((i%37)-18)*0.01; scale f16(0.02); q=trunc8(bi*5+t*3)
    m, n, k = 2, 5, 8192 + 64
    kb = k // 32
    a = (((np.arange(m * k) % 37) - 18) * 0.01).astype(np.float32).reshape(m, k)
    blocks = np.zeros((kb * n, 34), np.uint8)
    blocks[:, 0:2] = np.array([0.02], np.float16).view(np.uint8)
    bi = np.arange(kb * n, dtype=np.uint64)[:, None]
    t = np.arange(32, dtype=np.uint64)[None, :]
    blocks[:, 2:] = ((bi * np.uint64(5) + t * np.uint64(3)) & np.uint64(0xFF)).astype(np.uint8)
    got = orc.matmul_q8_kmajor(a, blocks, n)
    aq, a_s = np_prepare_a(a)
    b3 = blocks.reshape(kb, n, 34).transpose(1, 0, 2).copy()
    wq, w_s = split_q8(b3, n, kb)
    want = f64_formula(aq, a_s, wq, w_s)
    assert np.allclose(got, want, rtol=1e-5, atol=0)


@pytest.mark.parametrize("m", [1, 2, 5])
def test_nt_reference_style_inputs(orc, m):
    # matmul_nt_q.zig:587-637 compares against the f64 formula at abs 1e-4*max(1,|want|)
    rng = np.random.default_rng(11 + m)
    n, k = 13, 160
    w = (rng.standard_normal((n, k)) * 0.5).astype(np.float32)
    a = rng.standard_normal((m, k)).astype(np.float32)
    blocks = orc.quantize(orc.Q8_0, w, 1)
    got = orc.matmul_nt_q8(a, blocks, n)
    aq, a_s = np_prepare_a(a)
    wq, w_s = split_q8(blocks, n, k // 32)
    want = f64_formula(aq, a_s, wq, w_s)
    assert (np.abs(got - want) <= 1e-4 * np.maximum(1.0, np.abs(want))).all()
    assert np.allclose(got, want, rtol=2e-6, atol=1e-6)


@pytest.mark.parametrize("dt_name", ["q8", "q4"])
def test_lossless_activation_reduces_to_dequant_matmul(orc, dt_name):
    # A integer-valued with |a| max 127 in every block -> a_s = 1, aq = a: the int8 path must
    # equal A @ dequant(W) (textbook), which pins scales, nibble order and block addressing.
    rng = np.random.default_rng(21)
    m, n, k = 3, 9, 128
    a = rng.integers(-127, 128, (m, k)).astype(np.float32)
    a[:, ::32] = 127.0
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    dt = orc.Q8_0 if dt_name == "q8" else orc.Q4_0
    blocks = orc.quantize(dt, w, 0)                      # [K,N] axis 0 (K-major)
    deq = orc.dequantize(dt, blocks, (k, n), 0)
    want = a.astype(np.float64) @ deq.astype(np.float64)
    got_p = orc.matmul_q_packed(dt, a, blocks, n, kc=64)
    assert np.allclose(got_p, want, rtol=1e-5, atol=1e-5)
    f32a = orc.matmul_q_f32a(dt, False, a, blocks, n)
    assert np.allclose(f32a, want, rtol=1e-6, atol=1e-6)
    if dt_name == "q8":
        got_k = orc.matmul_q8_kmajor(a, blocks, n)
        assert np.allclose(got_k, want, rtol=1e-5, atol=1e-5)
        nt_blocks = blocks.reshape(k // 32, n, 34).transpose(1, 0, 2).copy()
        got_nt = orc.matmul_nt_q8(a, nt_blocks, n)
        assert np.array_equal(got_nt, got_k)             # same arithmetic, different block addressing


@pytest.mark.parametrize("dt_name", ["q8", "q4"])
def test_packed_matches_f64_formula_and_kc_is_only_summation_order(orc, dt_name):
    rng = np.random.default_rng(31)
    m, n, k = 4, 17, 512
    a = rng.standard_normal((m, k)).astype(np.float32)
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    dt = orc.Q8_0 if dt_name == "q8" else orc.Q4_0
    blocks = orc.quantize(dt, w, 0)
    bb = orc.BLOCK_BYTES[dt]
    b3 = blocks.reshape(k // 32, n, bb).transpose(1, 0, 2).copy()
    wq, w_s = (split_q8 if dt_name == "q8" else split_q4)(b3, n, k // 32)
    aq, a_s = np_prepare_a(a)
    want = f64_formula(aq, a_s, wq, w_s)
    outs = [orc.matmul_q_packed(dt, a, blocks, n, kc=kc) for kc in (128, 256, 512)]
    for o in outs:
        assert np.allclose(o, want, rtol=1e-5, atol=1e-6)
    # reference tolerance vs the plain f32 product (test_cpu_kernels.zig:572-617: abs 0.2 / 0.8)
    plain = a @ w
    assert np.abs(outs[1] - plain).max() < (0.2 if dt_name == "q8" else 0.8)


def test_alpha_beta_and_threads(orc):
    rng = np.random.default_rng(41)
    m, n, k = 2, 40, 96
    a = rng.standard_normal((m, k)).astype(np.float32)
    w = (rng.standard_normal((n, k)) * 0.1).astype(np.float32)
    c0 = rng.standard_normal((m, n)).astype(np.float32)
    blocks = orc.quantize(orc.Q8_0, w, 1)
    base = orc.matmul_nt_q8(a, blocks, n)
    got = orc.matmul_nt_q8(a, blocks, n, alpha=0.5, beta=2.0, c=c0)
    assert np.allclose(got, np.float32(0.5) * base + np.float32(2.0) * c0, rtol=1e-6, atol=1e-6)
    assert np.array_equal(orc.matmul_nt_q8(a, blocks, n, threads=4), base)   # partition never changes a result
    kb = orc.quantize(orc.Q4_0, np.ascontiguousarray(w.T), 0)
    p1 = orc.matmul_q_packed(orc.Q4_0, a, kb, n, alpha=0.5, beta=2.0, c=c0, kc=32)
    p0 = orc.matmul_q_packed(orc.Q4_0, a, kb, n, kc=32)
    assert np.allclose(p1, 0.5 * p0 + 2.0 * c0, rtol=1e-5, atol=1e-5)
    assert np.array_equal(orc.matmul_q_packed(orc.Q4_0, a, kb, n, kc=32, threads=3), p0)


def test_activation_quant_noise_floor_vs_f32a(orc):
    # the int8-A path differs from the f32-A dequant path by the activation-quant noise only:
    # NMSE ~ 3e-5 on N(0,0.02) weights x N(0,1) activations, independent of K
    rng = np.random.default_rng(51)
    n, k = 64, 2048
    a = rng.standard_normal((1, k)).astype(np.float32)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    blocks = orc.quantize(orc.Q8_0, w, 1)
    i8 = orc.matmul_nt_q8(a, blocks, n)
    f32a = orc.matmul_q_f32a(orc.Q8_0, True, a, blocks, n)
    nmse = float(((i8 - f32a) ** 2).sum() / (f32a ** 2).sum())
    assert 1e-6 < nmse < 2e-4


def test_prepare_a_hand_computed_ties_and_special_blocks(orc):
    # aion cpu/kernels/matmul_q_i8.zig:187-203 on blocks whose codes follow by hand: exact ties (Zig @round is half away
    # from zero), amax on a negative element, 127 / amax (not 1 / (amax / 127)), a zero block, a denormal amax whose
    # inverse overflows (every nonzero element then clamps to +-127)
    import act_cases as ac
    a = np.concatenate([np.array(ac.TIE_BLOCK, np.float32), np.array(ac.HALF_BLOCK, np.float32),
                        ac.block_kinds(np.random.default_rng(0))[3], np.zeros(32, np.float32),
                        ac.block_kinds(np.random.default_rng(0))[4]]).reshape(1, -1)
    aq, sc, sm = orc.prepare_a(a)
    aq = aq.reshape(5, 32)
    assert aq[0].tolist() == ac.TIE_CODES and sc[0, 0] == np.float32(1.0)
    half = [-127] + [(k + 1) * (1 if k % 2 else -1) for k in range(31)]          # (2k+1)/2 -> k+1, sign kept
    assert aq[1].tolist() == half and sc[0, 1] == np.float32(2.0)
    assert aq[2, :len(ac.INV_CODES)].tolist() == ac.INV_CODES
    assert not aq[3].any() and sc[0, 3] == 0.0
    assert aq[4].tolist() == [127 * (-1 if t % 2 else 1) for t in range(32)]
    assert sc[0, 4] == np.float32(5e-40) / np.float32(127) and sc[0, 4] > 0
    assert sm[0].tolist() == aq.astype(np.int64).sum(axis=1).tolist()


def test_matmul_nt_f32_restatement_against_float64_and_exact_inputs(orc):
    """MatMulNT with an f32 B (cpu/kernels/matmul_nt.zig:40-126). Pinned two ways: (1) inputs of small integers, where every
    product and every partial sum is an integer below 2^24 and so exact in f32 - ANY order of the additions gives the same
    bits, so the result must equal the integer matmul, alpha / beta included (a dropped tail element, a transposed operand or
    a wrong reduce shows); (2) random inputs against the float64 product within the worst-case bound of an f32 sum of K
    terms, gamma_K * sum|a||b|."""
    rng = np.random.default_rng(61)
    for m, n, k in [(1, 7, 1), (3, 5, 31), (2, 9, 32), (4, 6, 100), (1, 3, 4099)]:
        a = rng.integers(-8, 9, (m, k)).astype(np.float32)
        b = rng.integers(-8, 9, (n, k)).astype(np.float32)
        c0 = rng.integers(-4, 5, (m, n)).astype(np.float32)
        want = a.astype(np.int64) @ b.astype(np.int64).T
        assert np.array_equal(orc.matmul_nt_f32(a, b), want.astype(np.float32))
        assert np.array_equal(orc.matmul_nt_f32(a, b, alpha=2.0, beta=-0.5, c=c0), (2 * want - 0.5 * c0).astype(np.float32))
        # a different lane count is a different admissible order: same bits on exact inputs
        assert np.array_equal(orc.matmul_nt_f32(a, b, lanes=4), want.astype(np.float32))
    for m, n, k in [(2, 33, 64), (5, 17, 1000), (1, 8, 4096)]:
        a = rng.standard_normal((m, k)).astype(np.float32)
        b = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
        got = orc.matmul_nt_f32(a, b, alpha=0.75)
        ref = 0.75 * (a.astype(np.float64) @ b.astype(np.float64).T)
        bound = (k + 2) * 2.0 ** -24 * 0.75 * (np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64).T)
        assert (np.abs(got - ref) <= bound).all()
    with pytest.raises(ValueError):
        orc.matmul_nt_f32(np.zeros((1, 4), np.float32), np.zeros((2, 4), np.float32), beta=1.0)      # beta without C
