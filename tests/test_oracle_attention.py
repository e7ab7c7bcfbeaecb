"""Pins the oracle's attention and glue ops (CPU only).

Checks: textbook f64 attention, torch's scaled_dot_product_attention on the causal/GQA case,
the reference's hand-computable known answers (api/test_api.zig:3256-3331,
api/test_nn.zig:799-901), split == unsplit, window == equivalent mask, closed forms for the
approximations (|rel err| of exp <= t^5/120) and for rmsnorm / rope / gelu / argmax.
"""
import math

import numpy as np
import pytest


def np_attention(q, k, v, scale, lo_hi):
    """q [L,Hq,D], k/v [T,Hkv,D]; lo_hi(l) -> (lo,hi). float64 textbook."""
    L, Hq, D = q.shape
    Hkv = k.shape[1]
    g = Hq // Hkv
    out = np.zeros((L, Hq, v.shape[2]))
    for l in range(L):
        lo, hi = lo_hi(l)
        if hi <= lo:
            continue
        for h in range(Hq):
            s = (k[lo:hi, h // g].astype(np.float64) @ q[l, h].astype(np.float64)) * scale
            p = np.exp(s - s.max())
            out[l, h] = (p / p.sum()) @ v[lo:hi, h // g].astype(np.float64)
    return out


def test_exp_and_tanh_approx_error_bounds(orc):
    xs = np.linspace(-80, 0, 4001)
    rel = max(abs(orc.exp_approx(x) / math.exp(x) - 1) for x in xs)
    assert rel < 7e-5                       # t^5/120 at t = 0.347 (4.2e-5) plus f32 rounding of x/ln2 near -80
    assert orc.exp_approx(0.0) == 1.0
    assert max(abs(orc.tanh_approx(x) - math.tanh(x)) for x in np.linspace(-6, 6, 1201)) < 2e-4


@pytest.mark.parametrize("kv_dtype", [np.float32, np.float16])
def test_blocked_matches_f64_causal_gqa(orc, kv_dtype):
    rng = np.random.default_rng(7)
    B, L, Hq, Hkv, D = 2, 70, 8, 2, 64
    q = rng.standard_normal((B, L, Hq, D)).astype(np.float32)
    k = rng.standard_normal((B, L, Hkv, D)).astype(kv_dtype)
    v = rng.standard_normal((B, L, Hkv, D)).astype(kv_dtype)
    scale = 1 / math.sqrt(D)
    ref = orc.attention_f64(q, k, v, scale)
    got = orc.attention_blocked(q, k, v, scale)
    assert np.abs(got - ref).max() < 2e-4
    for b in range(B):
        want = np_attention(q[b], k[b].astype(np.float32), v[b].astype(np.float32), scale, lambda l: (0, l + 1))
        assert np.abs(ref[b] - want).max() < 1e-6


def test_f64_matches_torch_sdpa(orc):
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(8)
    B, L, Hq, Hkv, D = 1, 33, 8, 1, 32
    q = rng.standard_normal((B, L, Hq, D)).astype(np.float32)
    k = rng.standard_normal((B, L, Hkv, D)).astype(np.float32)
    v = rng.standard_normal((B, L, Hkv, D)).astype(np.float32)
    ref = orc.attention_f64(q, k, v, 1 / math.sqrt(D))
    tq, tk, tv = (torch.from_numpy(x).permute(0, 2, 1, 3).double() for x in (q, k, v))
    tk = tk.repeat_interleave(Hq // Hkv, dim=1)
    tv = tv.repeat_interleave(Hq // Hkv, dim=1)
    want = F.scaled_dot_product_attention(tq, tk, tv, is_causal=True).permute(0, 2, 1, 3).numpy()
    assert np.abs(ref - want).max() < 1e-6


def test_kat_uniform_softmax_sliding_window(orc):
    # api/test_api.zig:3256-3331: all-zero q,k -> uniform softmax over sliding(2,0); q [1,2,4,2],
    # kv [1,6,2,.], positions (4,5), end 6 -> {4,4,40,40,5,5,50,50}
    q = np.zeros((1, 2, 4, 2), np.float32)
    k = np.zeros((1, 6, 2, 2), np.float32)
    v = np.zeros((1, 6, 2, 1), np.float32)
    for t in range(6):
        v[0, t, 0, 0] = t + 1
        v[0, t, 1, 0] = 10 * (t + 1)
    pos = np.array([[4, 5]], np.int32)
    end = np.array([6], np.int32)
    for fn in (orc.attention_blocked, orc.attention_f64):
        out = fn(q, k, v, 1.0, window=(2, 0, 0), positions=pos, kv_lengths=end)
        assert np.allclose(out.reshape(-1), [4, 4, 40, 40, 5, 5, 50, 50], atol=1e-6)


def test_kat_three_step_decode(orc):
    # api/test_nn.zig:799-901: 1 head, 1 dim; step i appends k=v=(i+2)... expected 2, then
    # (e^-3*2+3)/(e^-3+1), then (e^-8*2+e^-4*3+4)/(e^-8+e^-4+1): scores q*k with q=k chosen so
    # s differences are -3 and -8,-4. Use q_t = k_t = v_t = t+2 at scale 1:
    # step 2 scores: 3*2=6, 3*3=9 -> diff -3; step 3: 4*2=8, 4*3=12, 4*4=16 -> diffs -8,-4.
    kc = np.zeros((1, 3, 1, 1), np.float32)
    vc = np.zeros((1, 3, 1, 1), np.float32)
    want = [2.0, (math.exp(-3) * 2 + 3) / (math.exp(-3) + 1),
            (math.exp(-8) * 2 + math.exp(-4) * 3 + 4) / (math.exp(-8) + math.exp(-4) + 1)]
    for t in range(3):
        kc[0, t, 0, 0] = vc[0, t, 0, 0] = t + 2
        q = np.full((1, 1, 1, 1), t + 2, np.float32)
        out = orc.attention_blocked(q, kc, vc, 1.0, positions=np.array([[t]], np.int32), kv_lengths=np.array([t + 1], np.int32))
        assert abs(float(out.reshape(-1)[0]) - want[t]) < 1e-4


def test_split_merge_equals_unsplit_and_window_equals_mask(orc):
    rng = np.random.default_rng(9)
    B, T, Hq, Hkv, D = 2, 700, 8, 1, 32
    q = rng.standard_normal((B, 1, Hq, D)).astype(np.float32)
    k = rng.standard_normal((B, T, Hkv, D)).astype(np.float16)
    v = rng.standard_normal((B, T, Hkv, D)).astype(np.float16)
    pos = np.array([[T - 1], [400]], np.int32)
    end = np.array([T, 401], np.int32)
    one = orc.attention_blocked(q, k, v, 0.2, positions=pos, kv_lengths=end, segs=1)
    four = orc.attention_blocked(q, k, v, 0.2, positions=pos, kv_lengths=end, segs=4)
    assert np.abs(one - four).max() < 1e-5
    # sliding window == explicit interval in the textbook reference
    win = orc.attention_blocked(q, k, v, 0.2, window=(100, 0, 0), positions=pos, kv_lengths=end)
    for b in range(B):
        p = int(pos[b, 0])
        want = np_attention(q[b], k[b].astype(np.float32), v[b].astype(np.float32), 0.2, lambda l: (p - 100, p + 1))
        assert np.abs(win[b] - want).max() < 2e-4
    # chunked window: anchor at chunk start
    ch = orc.attention_f64(q, k, v, 0.2, window=(16, 0, 64), positions=pos, kv_lengths=end)
    for b in range(B):
        p = int(pos[b, 0]); a = (p // 64) * 64
        want = np_attention(q[b], k[b].astype(np.float32), v[b].astype(np.float32), 0.2, lambda l: (a - 16, min(int(end[b]), a + 64)))
        assert np.abs(ch[b] - want).max() < 1e-6


def test_empty_window_gives_zeros(orc):
    q = np.ones((1, 1, 2, 4), np.float32)
    k = np.ones((1, 4, 1, 4), np.float32)
    v = np.ones((1, 4, 1, 4), np.float32)
    out = orc.attention_blocked(q, k, v, 1.0, kv_lengths=np.array([0], np.int32))
    assert not out.any()


def test_soft_cap(orc):
    rng = np.random.default_rng(10)
    q = rng.standard_normal((1, 5, 2, 16)).astype(np.float32) * 3
    k = rng.standard_normal((1, 5, 1, 16)).astype(np.float32) * 3
    v = rng.standard_normal((1, 5, 1, 16)).astype(np.float32)
    a = orc.attention_blocked(q, k, v, 1.0, soft_cap=5.0)
    b = orc.attention_f64(q, k, v, 1.0, soft_cap=5.0)
    assert np.abs(a - b).max() < 5e-3     # tanh approximation (1e-4 abs) times cap


def test_glue_closed_forms(orc):
    rng = np.random.default_rng(12)
    x = rng.standard_normal((3, 64)).astype(np.float32)
    g = rng.standard_normal(64).astype(np.float32)
    r = rng.standard_normal((3, 64)).astype(np.float32)
    want = x / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + 1e-6) * g
    assert np.allclose(orc.rmsnorm(x, g, 1e-6), want, rtol=1e-5, atol=1e-6)
    assert np.allclose(orc.rmsnorm(x, g, 1e-6, residual=r), want + r, rtol=1e-5, atol=1e-6)

    xr = rng.standard_normal((1, 4, 2, 8)).astype(np.float32)
    pos = np.array([[0, 1, 7, 100]], np.int32)
    got = orc.rope(xr, pos, base=10000.0)
    assert np.array_equal(got[0, 0], xr[0, 0])                     # position 0 is the identity
    D = 8
    for ti, p in enumerate(pos[0]):
        for i in range(D // 2):
            ang = p * 10000.0 ** (-2.0 * i / D)
            c, s = math.cos(ang), math.sin(ang)
            for h in range(2):
                xl, xr_ = xr[0, ti, h, i], xr[0, ti, h, i + D // 2]
                assert abs(got[0, ti, h, i] - (xl * c - xr_ * s)) < 2e-4
                assert abs(got[0, ti, h, i + D // 2] - (xl * s + xr_ * c)) < 2e-4
    norms_in = np.linalg.norm(xr, axis=3)
    assert np.allclose(np.linalg.norm(got, axis=3), norms_in, rtol=1e-5)   # rotations preserve norm

    a = rng.standard_normal(100).astype(np.float32) * 3
    b = rng.standard_normal(100).astype(np.float32)
    gelu = 0.5 * a * (1 + np.tanh(0.7978845608028654 * (a + 0.044715 * a ** 3)))
    assert np.allclose(orc.gate_gelu(a, b), gelu * b, atol=5e-4)

    z = np.array([[1, 5, 5, 2], [-1, -1, -3, -1]], np.float32)
    assert list(orc.argmax(z)) == [1, 0]                           # first maximum wins

    t = (rng.standard_normal((6, 64)) * 0.3).astype(np.float32)
    blk = orc.quantize(orc.Q8_0, t, 1)
    ids = np.array([5, 0, 5], np.int32)
    assert np.array_equal(orc.gather_rows(blk, ids, 64, dtype=orc.Q8_0), orc.dequantize(orc.Q8_0, blk, (6, 64), 1)[ids])
    assert np.array_equal(orc.gather_rows(t, ids, 64), t[ids])
    assert np.array_equal(orc.cast_f32_f16(t), t.astype(np.float16))
