"""GPU parity of the per-token glue steps against the CPU oracle (through the C ABI)."""
import numpy as np
import pytest

from aion_amd import backend as be
from aion_amd import hip

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,cols", [(5, 2048), (1, 2048), (3, 7), (2, 100), (4, 256), (2, 2049), (3, 4096)])
def test_rmsnorm_with_and_without_residual(gpu, orc, rows, cols):
    """Rows of up to 2048 columns run on the kernel that holds the row in registers, longer ones on the two-pass one."""
    rng = np.random.default_rng(1)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    g = rng.standard_normal(cols).astype(np.float32)
    bt = rng.standard_normal(cols).astype(np.float32)
    r = rng.standard_normal((rows, cols)).astype(np.float32)
    xb, gb, bb, rb = gpu.upload(x), gpu.upload(g), gpu.upload(bt), gpu.upload(r)
    out = gpu.alloc(x.nbytes)
    gpu.step_rmsnorm(out, xb, gb, rows, cols, 1e-6)
    assert np.allclose(gpu.download(out, np.float32, x.shape), orc.rmsnorm(x, g, 1e-6), rtol=1e-5, atol=1e-5)
    gpu.step_rmsnorm(out, xb, gb, rows, cols, 1e-6, beta=bb, residual=rb)
    assert np.allclose(gpu.download(out, np.float32, x.shape), orc.rmsnorm(x, g, 1e-6, beta=bt, residual=r), rtol=1e-5, atol=1e-5)  # three-term sum: fused multiply-add vs separate rounding
    want = orc.rmsnorm(x, g, 1e-6, beta=bt, residual=r)
    gpu.step_rmsnorm(rb, xb, gb, rows, cols, 1e-6, beta=bb, residual=rb)          # summed into the residual in place
    assert np.array_equal(gpu.download(rb, np.float32, x.shape), gpu.download(out, np.float32, x.shape))
    assert np.allclose(gpu.download(rb, np.float32, x.shape), want, rtol=1e-5, atol=1e-5)
    with pytest.raises(be.AionHipError) as e:
        gpu.step_rmsnorm(out, xb, gb, rows, cols, 0.0)
    assert e.value.status == hip.INVALID_ARGUMENT
    for b in (xb, gb, bb, rb, out):
        b.free()


@pytest.mark.parametrize("proportion", [1.0, 0.5, 0.0])
def test_rope_matches_oracle(gpu, orc, proportion):
    rng = np.random.default_rng(2)
    B, T, H, D = 2, 7, 8, 256
    x = rng.standard_normal((B, T, H, D)).astype(np.float32)
    pos = rng.integers(0, 5000, (B, T)).astype(np.int32)
    pos[0, 0] = 0
    xb, pb = gpu.upload(x), gpu.upload(pos)
    out = gpu.alloc(x.nbytes)
    gpu.step_rope(out, xb, pb, B, T, H, D, base=10000.0, proportion=proportion)
    got = gpu.download(out, np.float32, x.shape)
    want = orc.rope(x, pos, base=10000.0, proportion=proportion)
    assert np.allclose(got, want, rtol=0, atol=2e-6)
    assert np.array_equal(got[0, 0], x[0, 0])
    for b in (xb, pb, out):
        b.free()


def test_add_gate_cast_argmax(gpu, orc):
    rng = np.random.default_rng(3)
    n = 8192 + 5
    a = (rng.standard_normal(n) * 3).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    ab, bb = gpu.upload(a), gpu.upload(b)
    out = gpu.alloc(n * 4)
    gpu.step_add(out, ab, bb, n)
    assert np.array_equal(gpu.download(out, np.float32, (n,)), a + b)
    gpu.step_gate_gelu(out, ab, bb, n)
    assert np.allclose(gpu.download(out, np.float32, (n,)), orc.gate_gelu(a, b), rtol=1e-5, atol=1e-6)
    h = gpu.alloc(n * 2)
    gpu.step_cast_f32_f16(h, ab, n)
    assert np.array_equal(gpu.download(h, np.float16, (n,)), a.astype(np.float16))

    rows, m = 3, 262144
    x = rng.standard_normal((rows, m)).astype(np.float32)
    x[0, 1000] = x[0, 200000] = 50.0          # tie: the first maximum wins
    x[1, 0] = 60.0
    x[2, m - 1] = 70.0
    xb = gpu.upload(x)
    idx = gpu.alloc(rows * 4)
    gpu.step_argmax(idx, xb, rows, m)
    got = gpu.download(idx, np.int32, (rows,))
    assert list(got) == list(orc.argmax(x)) == [1000, 0, m - 1]
    for t in (ab, bb, out, h, xb, idx):
        t.free()


def test_gather_rows_f32_and_q8(gpu, orc):
    rng = np.random.default_rng(4)
    V, D = 50, 128
    table = (rng.standard_normal((V, D)) * 0.3).astype(np.float32)
    ids = np.array([49, 0, 7, 7, 13], np.int32)
    ib = gpu.upload(ids)
    out = gpu.alloc(ids.size * D * 4)
    tb = gpu.upload(table)
    gpu.step_gather_rows(be.F32, out, tb, ib, ids.size, D, V)
    assert np.array_equal(gpu.download(out, np.float32, (ids.size, D)), table[ids])
    blocks = be.quantize_blocks(be.Q8_0, table, 1)
    qb = gpu.upload(blocks)
    gpu.step_gather_rows(be.Q8_0, out, qb, ib, ids.size, D, V)
    assert np.array_equal(gpu.download(out, np.float32, (ids.size, D)), orc.gather_rows(blocks, ids, D, dtype=orc.Q8_0))
    for t in (ib, out, tb, qb):
        t.free()


def test_kv_append_f16_at_device_write_index(gpu, orc):
    rng = np.random.default_rng(5)
    B, S, T, H, D = 2, 3, 10, 1, 64
    cache = np.zeros((B, T, H, D), np.float16)
    cb = gpu.upload(cache)
    for step, widx in enumerate([(0, 4), (3, 0), (6, 7)]):           # one write index per batch entry
        src = rng.standard_normal((B, S, H, D)).astype(np.float32)
        sb, wb = gpu.upload(src), gpu.upload(np.array(widx, np.int32))
        gpu.step_append_f16(cb, sb, wb, B, S, T, H * D)
        cache = orc.sequence_append(cache, orc.cast_f32_f16(src), widx)
        assert np.array_equal(gpu.download(cb, np.float16, cache.shape), cache)
        sb.free(); wb.free()
    # a write index that would run past the capacity writes only what fits
    src = np.ones((B, S, H, D), np.float32)
    sb, wb = gpu.upload(src), gpu.upload(np.array([8, 8], np.int32))
    gpu.step_append_f16(cb, sb, wb, B, S, T, H * D)
    cache[:, 8:10] = 1.0
    assert np.array_equal(gpu.download(cb, np.float16, cache.shape), cache)
    for t in (cb, sb, wb):
        t.free()


def test_kv_append_into_a_rolling_cache(gpu, orc):
    rng = np.random.default_rng(8)
    B, T, H, D = 2, 12, 2, 32
    cache = np.zeros((B, T, H, D), np.float16)
    cb = gpu.upload(cache)
    t0 = np.array([0, 30], np.int32)
    for n in (5, 9, 1, 12, 7):
        src = rng.standard_normal((B, n, H, D)).astype(np.float32)
        sb, wb = gpu.upload(src), gpu.upload(t0)
        gpu.step_append_f16(cb, sb, wb, B, n, T, H * D, rolling=True)
        cache = orc.sequence_append(cache, orc.cast_f32_f16(src), t0, rolling=True)
        assert np.array_equal(gpu.download(cb, np.float16, cache.shape), cache)
        t0 = t0 + n
        sb.free(); wb.free()
    cb.free()


def test_argmax_ties_across_parts_and_repeated_launches(gpu, orc):
    """The row is cut into 64 parts whose (value, index) words meet behind a ticket: ties that span two parts (the smaller
    index wins whichever part's workgroup arrives last), a constant row (index 0), fewer elements than parts, negative
    rows, and the same launch repeated (the tickets return to zero)."""
    rng = np.random.default_rng(21)
    for m in (262144, 64 * 5 + 3, 40, 1):
        per = -(-m // 64)
        rows = 6
        x = rng.standard_normal((rows, m)).astype(np.float32)
        if m > 64:
            x[0, per - 1] = x[0, per] = 9.0                      # last element of part 0 and first of part 1
            x[1, 3 * per + 1] = x[1, min(40 * per + 2, m - 2)] = x[1, min(63 * per, m - 1)] = 11.0
            x[4, m - 1] = x[4, 0] = 12.0
        x[2, :] = -3.5                                        # constant: the first index
        x[3, :] = -np.abs(x[3, :]) - 1.0                      # all negative
        x[5, m // 2] = np.inf
        xb, idx = gpu.upload(x), gpu.alloc(rows * 4)
        want = list(orc.argmax(x))
        assert want == list(np.argmax(x, axis=1))
        for _ in range(5):
            gpu.step_argmax(idx, xb, rows, m)
            assert list(gpu.download(idx, np.int32, (rows,))) == want, m
        xb.free(); idx.free()


@pytest.mark.parametrize("np_dtype,dtype", [(np.float16, "F16"), (np.float32, "F32")])
def test_sequence_append_step_with_rows_of_the_cache_type(gpu, orc, np_dtype, dtype):
    """The step as the reference states it: rows already of the cache's element type, linear and rolling."""
    rng = np.random.default_rng(15)
    B, T, H, D = 2, 12, 2, 32
    for rolling in (False, True):
        cache = np.zeros((B, T, H, D), np_dtype)
        cb = gpu.upload(cache)
        t0 = np.array([0, 3 if not rolling else 30], np.int32)
        for n in (4, 1, 3) if not rolling else (5, 9, 1, 12, 7):
            src = rng.standard_normal((B, n, H, D)).astype(np_dtype)
            sb, wb = gpu.upload(src), gpu.upload(t0)
            gpu.step_sequence_append(getattr(be, dtype), cb, sb, wb, B, n, T, H * D, rolling=rolling)
            cache = orc.sequence_append(cache, src, t0, rolling=rolling)
            assert np.array_equal(gpu.download(cb, np_dtype, cache.shape), cache)
            t0 = t0 + n
            sb.free(); wb.free()
        cb.free()
    z = gpu.zeros(64)
    with pytest.raises(be.AionHipError):
        gpu.step_sequence_append(be.Q8_0, z, z, z, 1, 1, 1, 1)          # caches hold f16 or f32
    z.free()


def test_rope_append_equals_the_separate_steps(gpu, orc):
    rng = np.random.default_rng(6)
    B, S, T, Hq, Hkv, D = 2, 3, 12, 8, 1, 64
    q = rng.standard_normal((B, S, Hq, D)).astype(np.float32)
    k = rng.standard_normal((B, S, Hkv, D)).astype(np.float32)
    v = rng.standard_normal((B, S, Hkv, D)).astype(np.float32)
    pos = np.array([[4, 5, 6], [4, 5, 6]], np.int32)
    qb, kb, vb, pb, wb = gpu.upload(q), gpu.upload(k), gpu.upload(v), gpu.upload(pos), gpu.upload(np.array([4, 4], np.int32))
    qo = gpu.alloc(q.nbytes)
    kc, vc = gpu.zeros(B * T * Hkv * D * 2), gpu.zeros(B * T * Hkv * D * 2)
    gpu.step_rope_append(qo, qb, kb, vb, kc, vc, pb, wb, B, S, T, Hq, Hkv, D)
    assert np.allclose(gpu.download(qo, np.float32, q.shape), orc.rope(q, pos), atol=2e-6)
    want_k = np.zeros((B, T, Hkv, D), np.float16)
    want_v = np.zeros((B, T, Hkv, D), np.float16)
    want_k[:, 4:7] = orc.cast_f32_f16(orc.rope(k, pos))
    want_v[:, 4:7] = orc.cast_f32_f16(v)
    got_k = gpu.download(kc, np.float16, want_k.shape)
    assert np.allclose(got_k.astype(np.float32), want_k.astype(np.float32), atol=2e-3)   # f16 ulp at |x| < 4
    assert np.array_equal(gpu.download(vc, np.float16, want_v.shape), want_v)
    assert not got_k[:, :4].any() and not got_k[:, 7:].any()
    # and against this backend's own separate steps: identical arithmetic, identical bits
    qo2, kr = gpu.alloc(q.nbytes), gpu.alloc(k.nbytes)
    kc2 = gpu.zeros(B * T * Hkv * D * 2)
    gpu.step_rope(qo2, qb, pb, B, S, Hq, D)
    gpu.step_rope(kr, kb, pb, B, S, Hkv, D)
    gpu.step_append_f16(kc2, kr, wb, B, S, T, Hkv * D)
    assert np.array_equal(gpu.download(qo2, np.float32, q.shape), gpu.download(qo, np.float32, q.shape))
    assert np.array_equal(gpu.download(kc2, np.float16, want_k.shape), got_k)
    for t in (qb, kb, vb, pb, wb, qo, kc, vc, qo2, kr, kc2):
        t.free()


@pytest.mark.parametrize("B,S,T,Hq,Hkv,D,rolling,with_beta,proportion", [
    (1, 1, 16, 8, 1, 256, False, False, 1.0),      # one new token, the bench model's head shape
    (2, 3, 12, 4, 2, 64, False, True, 0.5),        # several tokens, two sequences, biased norms, half the pairs rotated
    (1, 5, 8, 4, 1, 128, True, False, 1.0),        # a ring: rows 6, 7, 0, 1, 2
    (1, 2, 9, 3, 3, 512, False, True, 1.0),        # the largest head size of the fused step
    (1, 1, 4, 2, 1, 6, True, False, 1.0),          # fewer pairs than lanes
])
def test_headnorm_rope_append_equals_the_separate_steps(gpu, orc, B, S, T, Hq, Hkv, D, rolling, with_beta, proportion):
    """Per-head RMSNorm(q, k, v) -> RoPE(q, k) -> f16 append(k, v) in one launch, against the oracle's separate steps
    (f32 rounding of the sum of squares, 1e-5) and against this backend's own, whose bits it reproduces."""
    rng = np.random.default_rng(B * 100 + D)
    q = rng.standard_normal((B, S, Hq, D)).astype(np.float32)
    k = rng.standard_normal((B, S, Hkv, D)).astype(np.float32)
    v = rng.standard_normal((B, S, Hkv, D)).astype(np.float32)
    gam = [(1 + 0.2 * rng.standard_normal(D)).astype(np.float32) for _ in range(3)]
    bet = [(0.1 * rng.standard_normal(D)).astype(np.float32) if with_beta else None for _ in range(3)]
    start = 6 if rolling and S > 1 else 3
    pos = np.tile(np.arange(start, start + S, dtype=np.int32), (B, 1))
    widx = np.full(B, start, np.int32)
    eps = 1e-6
    bufs = [gpu.upload(x) for x in (q, k, v, pos, widx)]
    qb, kb, vb, pb, wb = bufs
    gb = [gpu.upload(x) for x in gam]
    bb = [gpu.upload(x) if x is not None else None for x in bet]
    qo = gpu.alloc(q.nbytes)
    seed = rng.standard_normal((B, T, Hkv, D)).astype(np.float16)          # earlier rows must survive
    kc, vc = gpu.upload(seed), gpu.upload(seed)
    gpu.step_headnorm_rope_append(qo, qb, kb, vb, gb, bb, eps, kc, vc, pb, wb, B, S, T, Hq, Hkv, D, proportion=proportion, rolling=rolling)
    norm = lambda x, i: orc.rmsnorm(x.reshape(-1, D), gam[i], eps, beta=bet[i]).reshape(x.shape)
    want_q = orc.rope(norm(q, 0), pos, proportion=proportion)
    want_k = orc.cast_f32_f16(orc.rope(norm(k, 1), pos, proportion=proportion))
    want_v = orc.cast_f32_f16(norm(v, 2))
    rows = [(start + s) % T if rolling else start + s for s in range(S)]
    exp_k, exp_v = seed.copy(), seed.copy()
    exp_k[:, rows], exp_v[:, rows] = want_k, want_v
    got_q = gpu.download(qo, np.float32, q.shape)
    got_k, got_v = gpu.download(kc, np.float16, seed.shape), gpu.download(vc, np.float16, seed.shape)
    assert np.allclose(got_q, want_q, atol=1e-5, rtol=1e-5)
    assert np.allclose(got_k.astype(np.float32), exp_k.astype(np.float32), atol=4e-3)      # one f16 ulp at |x| < 8
    assert np.allclose(got_v.astype(np.float32), exp_v.astype(np.float32), atol=4e-3)
    untouched = [t for t in range(T) if t not in rows]
    assert np.array_equal(got_k[:, untouched], seed[:, untouched]) and np.array_equal(got_v[:, untouched], seed[:, untouched])
    # the separate steps of this backend on the same operands
    nq, nk, nv, q2, k2 = (gpu.alloc(x.nbytes) for x in (q, k, v, q, k))
    kc2, vc2 = gpu.upload(seed), gpu.upload(seed)
    for out, x, i, heads in ((nq, qb, 0, Hq), (nk, kb, 1, Hkv), (nv, vb, 2, Hkv)):
        gpu.step_rmsnorm(out, x, gb[i], B * S * heads, D, eps, beta=bb[i])
    gpu.step_rope(q2, nq, pb, B, S, Hq, D, proportion=proportion)
    gpu.step_rope(k2, nk, pb, B, S, Hkv, D, proportion=proportion)
    gpu.step_append_f16(kc2, k2, wb, B, S, T, Hkv * D, rolling=rolling)
    gpu.step_append_f16(vc2, nv, wb, B, S, T, Hkv * D, rolling=rolling)
    # identical arithmetic in the identical order: identical bits
    assert np.array_equal(gpu.download(q2, np.float32, q.shape), got_q)
    assert np.array_equal(gpu.download(kc2, np.float16, seed.shape), got_k)
    assert np.array_equal(gpu.download(vc2, np.float16, seed.shape), got_v)
    with pytest.raises(Exception):
        gpu.step_headnorm_rope_append(qo, qb, kb, vb, gb, bb, eps, kc, vc, pb, wb, B, S, T, Hq, Hkv, 1024)
    for t in bufs + gb + [x for x in bb if x is not None] + [qo, kc, vc, nq, nk, nv, q2, k2, kc2, vc2]:
        t.free()


@pytest.mark.parametrize("dtype", ["q4", "q8"])
@pytest.mark.parametrize("D,Hq,Hkv,K", [(256, 8, 1, 2048), (64, 4, 2, 512), (128, 8, 2, 5120), (64, 16, 4, 8192)])
def test_qkv_rope_append_fusion_equals_the_separate_steps(gpu, orc, dtype, D, Hq, Hkv, K):
    """RMSNorm -> q/k/v matmuls -> RoPE -> f16 append in one launch against the same steps issued one by one
    (and through them against the oracle, which the separate steps are tested against)."""
    from aion_amd import backend as be
    rng = np.random.default_rng(D + K)
    dt = be.Q4_0 if dtype == "q4" else be.Q8_0
    ws = []
    for n in (Hq * D, Hkv * D, Hkv * D):
        w = (rng.standard_normal((K, n)) * 0.05).astype(np.float32)
        ws.append(gpu.upload_weight(dt, be.KMAJOR_KN, n, K, be.quantize_blocks(dt, w, 0)))
    T, widx, pos = 9, 5, 37
    x = gpu.upload(rng.standard_normal((1, K)).astype(np.float32))
    gamma = gpu.upload((1 + 0.1 * rng.standard_normal(K)).astype(np.float32))
    pb, wb = gpu.upload(np.array([[pos]], np.int32)), gpu.upload(np.array([widx], np.int32))
    # separate steps
    q, k, v = gpu.alloc(Hq * D * 4), gpu.alloc(Hkv * D * 4), gpu.alloc(Hkv * D * 4)
    qr = gpu.alloc(Hq * D * 4)
    kc, vc = gpu.zeros(T * Hkv * D * 2), gpu.zeros(T * Hkv * D * 2)
    gpu.step_rmsnorm_matmul(ws, x, gamma, 1, [q, k, v], 1e-6)
    gpu.step_rope_append(qr, q, k, v, kc, vc, pb, wb, 1, 1, T, Hq, Hkv, D, proportion=0.75)
    # one launch
    qr2 = gpu.alloc(Hq * D * 4)
    kc2, vc2 = gpu.zeros(T * Hkv * D * 2), gpu.zeros(T * Hkv * D * 2)
    gpu.step_rmsnorm_qkv_rope_append(ws[0], ws[1], ws[2], x, gamma, 1e-6, qr2, kc2, vc2, pb, wb, T, Hq, Hkv, D, proportion=0.75)
    assert gpu.last_kernel() == "gemv_%s_rmsnorm_rope" % dtype
    a, b2 = gpu.download(qr, np.float32, (Hq, D)), gpu.download(qr2, np.float32, (Hq, D))
    # same integer dots and scales; only the f32 summation order over lanes differs between 1 and 8 rows per wavefront
    assert np.abs(a - b2).max() <= 1e-5 * np.sqrt((a ** 2).mean())
    ka, kb2 = gpu.download(kc, np.float16, (T, Hkv, D)), gpu.download(kc2, np.float16, (T, Hkv, D))
    va, vb2 = gpu.download(vc, np.float16, (T, Hkv, D)), gpu.download(vc2, np.float16, (T, Hkv, D))
    assert np.abs(ka.astype(np.float32) - kb2.astype(np.float32)).max() <= 2e-3 * max(1.0, np.abs(ka.astype(np.float32)).max())
    assert np.abs(va.astype(np.float32) - vb2.astype(np.float32)).max() <= 2e-3 * max(1.0, np.abs(va.astype(np.float32)).max())
    assert not kb2[:widx].any() and not kb2[widx + 1:].any() and kb2[widx].any()
    assert not vb2[:widx].any() and not vb2[widx + 1:].any() and vb2[widx].any()
    # a write index outside the cache writes nothing
    wb_bad = gpu.upload(np.array([T], np.int32))
    kc3, vc3 = gpu.zeros(T * Hkv * D * 2), gpu.zeros(T * Hkv * D * 2)
    gpu.step_rmsnorm_qkv_rope_append(ws[0], ws[1], ws[2], x, gamma, 1e-6, qr2, kc3, vc3, pb, wb_bad, T, Hq, Hkv, D)
    assert not gpu.download(kc3, np.float16, (T, Hkv, D)).any() and not gpu.download(vc3, np.float16, (T, Hkv, D)).any()
    # rolling caches: the same out-of-range step lands in row step % T, with the values the in-range write gave
    wb_ring = gpu.upload(np.array([3 * T + widx], np.int32))
    gpu.step_rmsnorm_qkv_rope_append(ws[0], ws[1], ws[2], x, gamma, 1e-6, qr2, kc3, vc3, pb, wb_ring, T, Hq, Hkv, D, proportion=0.75, rolling=True)
    assert np.array_equal(gpu.download(kc3, np.float16, (T, Hkv, D)), kb2) and np.array_equal(gpu.download(vc3, np.float16, (T, Hkv, D)), vb2)
    wb_ring.free()
    for t in (x, gamma, pb, wb, wb_bad, q, k, v, qr, kc, vc, qr2, kc2, vc2, kc3, vc3):
        t.free()
    for w in ws:
        w.free()


@pytest.mark.parametrize("dtype", ["q4", "q8"])
@pytest.mark.parametrize("K,F", [(2048, 8192), (256, 96), (4096, 1024), (5120, 1024), (8192, 2048)])
def test_geglu_fusion_equals_the_separate_steps(gpu, orc, dtype, K, F):
    """RMSNorm -> gate/up matmuls -> gelu gate -> int8 preparation -> down matmul in two launches against the
    separate steps: the prepared codes are the same integers, so the result is the same up to f32 summation order."""
    from aion_amd import backend as be
    rng = np.random.default_rng(K + F)
    dt = be.Q4_0 if dtype == "q4" else be.Q8_0
    mk = lambda n, k: gpu.upload_weight(dt, be.KMAJOR_KN, n, k, be.quantize_blocks(dt, (rng.standard_normal((k, n)) * 0.05).astype(np.float32), 0))
    wg, wu, wd = mk(F, K), mk(F, K), mk(K, F)
    xv = rng.standard_normal((1, K)).astype(np.float32)
    gamma = gpu.upload((1 + 0.1 * rng.standard_normal(K)).astype(np.float32))
    x1, x2 = gpu.upload(xv), gpu.upload(xv)
    g, u = gpu.alloc(F * 4), gpu.alloc(F * 4)
    gpu.step_rmsnorm_matmul([wg, wu], x1, gamma, 1, [g, u], 1e-6)
    gpu.step_gate_matmul(wd, g, u, 1, x1, beta=1.0)
    gpu.step_rmsnorm_geglu_matmul(wg, wu, wd, x2, gamma, 1e-6, x2, beta=1.0)
    assert gpu.last_kernel() == "gemv_%s" % dtype
    a, b2 = gpu.download(x1, np.float32, (K,)), gpu.download(x2, np.float32, (K,))
    # an f32 rounding difference in g or u can flip one int8 code of h: allow that much and no more
    assert np.abs(a - b2).max() <= 2e-3 * np.sqrt((a ** 2).mean())
    for t in (gamma, x1, x2, g, u):
        t.free()
    for w in (wg, wu, wd):
        w.free()


def test_stream_read_probe_runs_and_checks_its_arguments(gpu):
    # the measurement aid: reads only (the source and the sink stay as they were), 16-byte granularity enforced
    data = np.arange(1 << 18, dtype=np.uint32)
    src = gpu.upload(data)
    sink = gpu.upload(np.array([7, 7, 7, 7], np.uint32))
    gpu.profile_start()
    gpu.probe_stream_read(src, 0, data.nbytes, sink)
    gpu.probe_stream_read(src, 4096, 65536, sink)
    gpu.probe_stream_read(src, 0, 0, sink)                       # nothing to read: no launch
    prof = gpu.profile_stop()
    assert [nm for nm, _ in prof] == ["stream_read", "stream_read"]
    assert all(ms > 0 for _, ms in prof)
    assert (gpu.download(src, np.uint32, data.shape) == data).all()
    assert (gpu.download(sink, np.uint32, (4,)) == 7).all()
    for off, nb in ((8, 64), (0, 24)):
        with pytest.raises(be.AionHipError):
            gpu.probe_stream_read(src, off, nb, sink)
    src.free(); sink.free()


def test_cache_growth_golden_vectors(gpu):
    # storage/test_storage.zig:883-898: ring [4,5,0,3], end 6, 3 retained, grown to 7
    src, ends = gpu.upload(np.array([4, 5, 0, 3], np.float32)), gpu.upload(np.array([6], np.int32))
    dst = gpu.upload(np.full(7, 77, np.float32))
    gpu.cache_grow_rolling(dst, src, ends, 1, 4, 7, 4, 3)
    assert gpu.download(dst, np.float32, (7,)).tolist() == [0, 0, 0, 3, 4, 5, 0]
    # backend/cpu/test_cpu_backend.zig:4718-4790: [0,1,2,3] grown to 8, then [90,91] appended at 5 (here an f16 cache)
    old = gpu.upload(np.array([0, 1, 2, 3], np.float16))
    new = gpu.upload(np.full(8, 77, np.float16))
    gpu.cache_grow(new, old, 1, 8, 16)
    app, wi = gpu.upload(np.array([90, 91], np.float32)), gpu.upload(np.array([5], np.int32))
    gpu.step_append_f16(new, app, wi, 1, 2, 8, 1)
    assert gpu.download(new, np.float16, (8,)).tolist() == [0, 1, 2, 3, 0, 90, 91, 0]
    # storage/test_storage.zig:862-873 and the schedule's corner cases
    assert gpu.cache_grow_target(8, 2, 1) == 16 and gpu.cache_grow_target(3, 3, 2) == 5 and gpu.cache_grow_target(5, 1, 1) == 6
    with pytest.raises(ValueError):
        gpu.cache_grow_target(0, 2, 1)
    for t in (src, ends, dst, old, new, app, wi):
        t.free()


@pytest.mark.parametrize("B,T,new_T,H,D", [(1, 4, 16, 1, 2), (3, 7, 9, 2, 64), (2, 128, 512, 1, 256)])
def test_cache_growth_against_the_oracle(gpu, orc, B, T, new_T, H, D):
    rng = np.random.default_rng(11)
    cache = rng.standard_normal((B, T, H, D)).astype(np.float16)
    src = gpu.upload(cache)
    dst = gpu.upload(np.full((B, new_T, H, D), 7, np.float16))             # stale contents must not survive
    gpu.cache_grow(dst, src, B, T * H * D * 2, new_T * H * D * 2)
    assert np.array_equal(gpu.download(dst, np.float16, (B, new_T, H, D)), orc.grow_axis(cache, 1, new_T))
    for retained, ends in ((T, [T + 3] * B), (max(1, T // 2), list(range(1, 2 * T, max(1, (2 * T - 1) // B)))[:B]), (10 * T, [0] * B), (3, [5 * T + b for b in range(B)])):
        eb = gpu.upload(np.array(ends, np.int32))
        gpu.write(dst, np.full((B, new_T, H, D), 7, np.float16))
        gpu.cache_grow_rolling(dst, src, eb, B, T, new_T, H * D * 2, retained)
        assert np.array_equal(gpu.download(dst, np.float16, (B, new_T, H, D)), orc.grow_rolling(cache, new_T, retained, ends)), (retained, ends)
        eb.free()
    src.free(); dst.free()


def test_cache_growth_rejects_bad_arguments(gpu):
    from aion_amd.hip import AionHipError
    a, b, e = gpu.zeros(64), gpu.zeros(64), gpu.zeros(4)
    for call in (lambda: gpu.cache_grow(a, a, 1, 8, 16), lambda: gpu.cache_grow(a, b, 1, 16, 8), lambda: gpu.cache_grow(a, b, 1, 6, 16),
                 lambda: gpu.cache_grow_rolling(a, b, e, 1, 4, 4, 4, 3), lambda: gpu.cache_grow_rolling(a, b, e, 1, 0, 4, 4, 3),
                 lambda: gpu.cache_grow_rolling(a, b, e, 1, 4, 8, 6, 3), lambda: gpu.cache_grow_rolling(a, a, e, 1, 4, 8, 4, 3)):
        with pytest.raises(AionHipError):
            call()
    gpu.cache_grow(a, b, 0, 8, 16)          # nothing to do
    a.free(); b.free(); e.free()


def test_unary_and_binary_steps(gpu, orc):
    rng = np.random.default_rng(31)
    from aion_amd.hip import AionHipError
    x = np.concatenate([rng.standard_normal(5000).astype(np.float32) * 4, np.array([0, -0.0, 30, -30, 88, -88, 1e-6], np.float32)])
    xb, ob = gpu.upload(x), gpu.alloc(x.nbytes)
    for op in ("relu", "gelu", "silu", "sigmoid", "tanh", "sqrt"):
        src = np.abs(x) if op == "sqrt" else x
        gpu.write(xb, src)
        gpu.step_unary(op, ob, xb, x.size)
        got, want = gpu.download(ob, np.float32, x.shape), orc.unary(op, src)
        # the same exp polynomial and the same operations; only mul+add contraction may differ by an ulp or two
        assert np.abs(got - want).max() <= 4e-7 * max(1.0, float(np.abs(want).max())), op
    with pytest.raises(AionHipError):
        gpu.step_unary("log", ob, xb, x.size)
    a = rng.standard_normal((6, 5, 64)).astype(np.float32)
    ab, outb = gpu.upload(a), gpu.alloc(a.nbytes)
    for b in (rng.standard_normal((6, 5, 64)).astype(np.float32) + 3, np.array([0.37], np.float32), rng.standard_normal(64).astype(np.float32) + 3,
              rng.standard_normal((5, 64)).astype(np.float32) + 3):
        bb = gpu.upload(b)
        for op in ("add", "sub", "mul", "div"):
            gpu.step_binary(op, outb, ab, bb, a.size, b.size)
            assert np.array_equal(gpu.download(outb, np.float32, a.shape), orc.binary(op, a, b)), (op, b.shape)
        bb.free()
    bad = gpu.upload(np.ones(7, np.float32))
    with pytest.raises(AionHipError):
        gpu.step_binary("add", outb, ab, bad, a.size, 7)
    # in place
    gpu.step_binary("mul", ab, ab, ab, a.size)
    assert np.array_equal(gpu.download(ab, np.float32, a.shape), a * a)
    for t in (xb, ob, ab, outb, bad):
        t.free()


def test_advance_state_logs_tokens_at_a_device_index(gpu):
    """advance_state with a token log: the tokens land at the index the counter held BEFORE the step moved it (the index
    may be one of the counters), writes past the capacity are dropped, and the plain entry point is unchanged."""
    ids, tok = gpu.upload(np.array([0], np.int32)), gpu.upload(np.array([41], np.int32))
    pos, end = gpu.upload(np.array([3], np.int32)), gpu.upload(np.array([4], np.int32))
    log = gpu.upload(np.full(6, -1, np.int32))
    for step in range(4):                                   # positions 3, 4, 5 fit the log of 6, position 6 does not
        gpu.write(tok, np.array([41 + step], np.int32))
        gpu.step_advance_state(ids, tok, 1, [pos, end], log=log, log_index=pos, log_capacity=6)
    assert list(gpu.download(log, np.int32, (6,))) == [-1, -1, -1, 41, 42, 43]
    assert int(gpu.download(ids, np.int32, (1,))[0]) == 44
    assert int(gpu.download(pos, np.int32, (1,))[0]) == 7 and int(gpu.download(end, np.int32, (1,))[0]) == 8
    gpu.step_advance_state(ids, tok, 1, [pos])              # no log
    assert int(gpu.download(pos, np.int32, (1,))[0]) == 8
    assert list(gpu.download(log, np.int32, (6,))) == [-1, -1, -1, 41, 42, 43]
    for t in (ids, tok, pos, end, log):
        t.free()

