"""GPU parity of the attention step against the CPU oracle (through the C ABI).

Tolerances are relative and per output row (one head's values for one query: an average of values, which shrinks like
1/sqrt(visible keys), so an absolute bound would loosen with the cache length). The gate is the row's max relative error
in the maximum norm, max |err| / max |reference row|, worst row (conftest.row_rel_err): <= 2e-3 with f32 accumulation
over an f16 cache, <= 1e-2 with bf16 operands. Beside it the same error against the row's rms (conftest.row_rms_err, 2.5
to 3 times stricter) is printed and held to 1.5 times those bounds: the kernels round q and the probabilities to the
cache's element type for the MFMA, and a float64 model of exactly that rounding and nothing else gives 1.9e-3 to 2.3e-3
(f16) and 8e-3 to 9e-3 (bf16) for this statistic on the prompts below (it is the largest of 1e5..1e6 samples of rounding
noise); a dropped key segment or a wrong merge weight shows as O(1) in both.
The reference is the textbook f64 attention (orc.attention_f64); aion's blocked CPU algorithm
(orc.attention_blocked, polynomial exp) is compared as well at the same bound.
"""
import math
import sys

import numpy as np
import pytest

from aion_amd import backend as be
from conftest import row_rel_err, row_rms_err

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def attn_err(got, ref, tol, tag=""):
    """asserts the worst row's max relative error under `tol` and the rms form under 1.5 * tol (see the module text)"""
    e_max, e_rms = row_rel_err(got, ref), row_rms_err(got, ref)
    say("  %s worst row: max|err|/max|ref| = %.2e   max|err|/rms(ref) = %.2e   (bar %.0e)" % (tag, e_max, e_rms, tol))
    assert np.isfinite(np.asarray(got)).all() and e_max < tol and e_rms < 1.5 * tol, (tag, e_max, e_rms, tol)
    return e_max


def to_bf16(x):
    """round-to-nearest-even f32 -> bf16 bits (uint16) and the f32 value they stand for"""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    bits = u.astype(np.uint16)
    return bits, (bits.astype(np.uint32) << 16).view(np.float32)


def run_attention(gpu, q, k, v, scale, q_dtype, kv_dtype, window=be.CAUSAL, soft_cap=0.0, positions=None, kv_lengths=None, rolling=False):
    B, L, Hq, Dk = q.shape
    _, T, Hkv, _ = k.shape
    Dv = v.shape[3]
    bufs = [gpu.upload(q), gpu.upload(k), gpu.upload(v)]
    out = gpu.alloc(max(B * L * Hq * Dv * 4, 4))
    pos = gpu.upload(np.ascontiguousarray(positions, np.int32)) if positions is not None else None
    kl = gpu.upload(np.ascontiguousarray(kv_lengths, np.int32)) if kv_lengths is not None else None
    gpu.step_attention(out, bufs[0], bufs[1], bufs[2], (B, L, T, Hq, Hkv, Dk, Dv), scale, q_dtype=q_dtype, kv_dtype=kv_dtype,
                       window=window, soft_cap=soft_cap, query_positions=pos, kv_lengths=kl, rolling=rolling)
    res = gpu.download(out, np.float32, (B, L, Hq, Dv))
    for b in bufs + [out] + [x for x in (pos, kl) if x is not None]:
        b.free()
    return res


def make_qkv(seed, B, L, T, Hq, Hkv, D, kind):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((B, L, Hq, D)).astype(np.float32)
    k = rng.standard_normal((B, T, Hkv, D)).astype(np.float32)
    v = rng.standard_normal((B, T, Hkv, D)).astype(np.float32)
    if kind == "f16":      # aion's cached decode: q f32, K/V cache f16
        k16, v16 = k.astype(np.float16), v.astype(np.float16)
        return (q, k16, v16, be.F32, be.F16), (q, k16.astype(np.float32), v16.astype(np.float32))
    qb, qf = to_bf16(q); kb, kf = to_bf16(k); vb, vf = to_bf16(v)   # BASELINE config 4: bf16 Q/K/V
    return (qb, kb, vb, be.BF16, be.BF16), (qf, kf, vf)


# A prompt with few 128-row workgroups runs on the 16-row split kernel (up to about 80 / 40 / 32 of them at head size
# 64 / 128 / 256: the smaller the head, the longer the 16-row kernel stays ahead). L = 150 (2 x 2 units x 5 workgroups) is
# such a prompt at every head size, L = 560 (2 x 2 x 18 = 72) at head size 64 only, L = 1100 (140) at none.
@pytest.mark.parametrize("kind,tol", [("f16", 2e-3), ("bf16", 1e-2)])
@pytest.mark.parametrize("D,L,kernel", [(64, 150, "attn_flash_split"), (128, 150, "attn_flash_split"), (256, 150, "attn_flash_split"),
                                        (64, 560, "attn_flash_split"), (128, 560, "attn_prefill"), (256, 560, "attn_prefill"),
                                        (64, 1100, "attn_prefill")])
def test_prefill_causal_gqa(gpu, orc, kind, tol, D, L, kernel):
    B, Hq, Hkv = 2, 8, 2
    say("prefill", kind, D, L)
    (q, k, v, qd, kd), (qf, kf, vf) = make_qkv(D, B, L, L, Hq, Hkv, D, kind)
    got = run_attention(gpu, q, k, v, 1 / math.sqrt(D), qd, kd)
    assert gpu.last_kernel() == kernel
    ref = orc.attention_f64(qf, kf, vf, 1 / math.sqrt(D))
    attn_err(got, ref, tol)
    blocked = orc.attention_blocked(qf, kf, vf, 1 / math.sqrt(D))
    attn_err(got, blocked, tol)


def test_prefill_head_256_stale_tail_odd_lengths_and_scales(gpu, orc):
    """The head-size-256 prefill loop reads whole 64-key tiles by address arithmetic on a uniform tile base and takes
    the row maximum before the softmax scale: a cache longer than the lengths in use whose tail holds NaN patterns,
    lengths that end inside a tile, a large scale (scores far apart: the lazy reference maximum moves often), and a
    scale that is not positive, which the 16-row kernel takes instead."""
    B, L, T, Hq, Hkv, D = 2, 300, 1000, 8, 2, 256
    (q, k, v, qd, kd), (qf, kf, vf) = make_qkv(77, B, L, T, Hq, Hkv, D, "f16")
    ends = np.array([911, 333], np.int32)
    pos = np.stack([np.arange(e - L, e, dtype=np.int32) for e in ends])
    for b in range(B):
        k[b, ends[b]:] = np.nan
        v[b, ends[b]:] = np.nan
    # (the queries are rounded to f16 for the MFMA: the error of a score grows with the scale, hence the second bar)
    for scale, kernel, tol in ((1 / 16.0, "attn_prefill", 2e-3), (0.25, "attn_prefill", 8e-3), (-0.05, "attn_flash_split", 2e-3)):
        got = run_attention(gpu, q, k, v, scale, qd, kd, positions=pos, kv_lengths=ends)
        assert gpu.last_kernel() == kernel
        ref = orc.attention_f64(qf, kf, vf, scale, positions=pos, kv_lengths=ends)
        attn_err(got, ref, tol)


@pytest.mark.parametrize("kind,tol", [("f16", 2e-3), ("bf16", 1e-2)])
@pytest.mark.parametrize("T,B", [(1024, 1), (1024, 8), (4096, 1), (4096, 8), (16384, 1), (16384, 8), (777, 3)])
def test_decode_split_k(gpu, orc, kind, tol, T, B):
    # BASELINE config 4b, every (T, B) it names: 1 query token at position T-1, 8 q heads / 1 kv head, hd 256
    Hq, Hkv, D = 8, 1, 256
    say("decode", kind, T, B)
    (q, k, v, qd, kd), (qf, kf, vf) = make_qkv(T + B, B, 1, T, Hq, Hkv, D, kind)
    pos = np.full((B, 1), T - 1, np.int32)
    end = np.full((B,), T, np.int32)
    got = run_attention(gpu, q, k, v, 1 / 16.0, qd, kd, positions=pos, kv_lengths=end)
    assert gpu.last_kernel() == "attn_flash_split"
    ref = orc.attention_f64(qf, kf, vf, 1 / 16.0, positions=pos, kv_lengths=end)
    attn_err(got, ref, tol)


def test_decode_ragged_lengths_and_stale_cache_tail(gpu, orc):
    # per-batch kv lengths; the cache tail beyond each length holds NaN patterns that must not leak
    B, T, Hq, Hkv, D = 3, 600, 8, 2, 128
    (q, k, v, qd, kd), (qf, kf, vf) = make_qkv(5, B, 1, T, Hq, Hkv, D, "f16")
    lens = np.array([600, 37, 1], np.int32)
    pos = (lens - 1).reshape(B, 1)
    for b in range(B):
        k[b, lens[b]:] = np.float16(np.nan)
        v[b, lens[b]:] = np.float16(np.nan)
        kf[b, lens[b]:] = 0
        vf[b, lens[b]:] = 0
    got = run_attention(gpu, q, k, v, 0.1, qd, kd, positions=pos, kv_lengths=lens)
    ref = orc.attention_f64(qf, kf, vf, 0.1, positions=pos, kv_lengths=lens)
    assert np.isfinite(got).all()
    attn_err(got, ref, 2e-3)


@pytest.mark.parametrize("window", [(100, 0, 0), (16, 0, 64), (be.UNBOUNDED, be.UNBOUNDED, 0), (5, 3, 0)])
def test_windows_prefill_and_decode(gpu, orc, window):
    B, L, Hq, Hkv, D = 1, 200, 4, 1, 64
    say("window", window)
    (q, k, v, qd, kd), (qf, kf, vf) = make_qkv(11, B, L, L, Hq, Hkv, D, "f16")
    got = run_attention(gpu, q, k, v, 0.125, qd, kd, window=window)
    ref = orc.attention_f64(qf, kf, vf, 0.125, window=window)
    attn_err(got, ref, 2e-3)
    # one decode row with an explicit position inside the sequence
    pos = np.array([[131]], np.int32)
    end = np.array([180], np.int32)
    got1 = run_attention(gpu, q[:, :1], k, v, 0.125, qd, kd, window=window, positions=pos, kv_lengths=end)
    ref1 = orc.attention_f64(qf[:, :1], kf, vf, 0.125, window=window, positions=pos, kv_lengths=end)
    attn_err(got1, ref1, 2e-3)


def test_prefill_bf16_key_segments_empty_segments_and_value_range(gpu, orc):
    """Over a bf16 cache the key segments of the prefill kernel leave f16 partial accumulators under a per-row power-of-two
    scale. A sliding window leaves whole segments of a row tile without a visible key (empty partial results beside live
    ones), a short cache length cuts the last segments, and values of magnitude 2^100 and 2^-100 (exact in bf16) lie far
    outside what f16 holds without the scale."""
    B, L, Hq, Hkv, D = 1, 1024, 8, 1, 128
    (q, k, v, qd, kd), (qf, kf, vf) = make_qkv(77, B, L, L, Hq, Hkv, D, "bf16")
    pos = np.arange(L, dtype=np.int32).reshape(1, L)
    for window, lens in (((100, 0, 0), None), (be.CAUSAL, np.array([700], np.int32)), ((16, 0, 64), None)):
        say("bf16 key segments", window, lens)
        got = run_attention(gpu, q, k, v, 1 / math.sqrt(D), qd, kd, window=window, positions=pos, kv_lengths=lens)
        assert gpu.last_kernel() == "attn_prefill"
        ref = orc.attention_f64(qf, kf, vf, 1 / math.sqrt(D), window=window, positions=pos, kv_lengths=lens)
        attn_err(got, ref, 1e-2)
    ref = orc.attention_f64(qf, kf, vf, 1 / math.sqrt(D))
    for e in (100, -100):
        vb, vbf = to_bf16(vf * np.float32(2.0 ** e))
        got = run_attention(gpu, q, k, vb, 1 / math.sqrt(D), qd, kd)
        assert gpu.last_kernel() == "attn_prefill"
        attn_err(got * np.float32(2.0 ** -e), ref, 1e-2)


def test_soft_cap(gpu, orc):
    (q, k, v, qd, kd), (qf, kf, vf) = make_qkv(13, 1, 40, 40, 8, 1, 64, "f16")
    # logits of std ~24 before the cap: the flash kernel feeds q to the MFMA in the K/V element
    # type, so the reference gets the same f16-rounded q (the cap itself is what is under test)
    q3 = (q * 3).astype(np.float16).astype(np.float32)
    got = run_attention(gpu, q3, k, v, 1.0, qd, kd, soft_cap=5.0)
    ref = orc.attention_f64(q3, kf, vf, 1.0, soft_cap=5.0)
    attn_err(got, ref, 2e-3)


def test_kat_uniform_softmax_sliding_window(gpu):
    # aion api/test_api.zig:3256-3331 -> {4,4,40,40,5,5,50,50}, abs 1e-6 (generic kernel: d_k=2, f32 K/V)
    q = np.zeros((1, 2, 4, 2), np.float32)
    k = np.zeros((1, 6, 2, 2), np.float32)
    v = np.zeros((1, 6, 2, 1), np.float32)
    for t in range(6):
        v[0, t, 0, 0] = t + 1
        v[0, t, 1, 0] = 10 * (t + 1)
    got = run_attention(gpu, q, k, v, 1.0, be.F32, be.F32, window=(2, 0, 0), positions=np.array([[4, 5]], np.int32), kv_lengths=np.array([6], np.int32))
    assert gpu.last_kernel() == "attn_generic"
    assert np.allclose(got.reshape(-1), [4, 4, 40, 40, 5, 5, 50, 50], atol=1e-6)


def test_kat_three_step_decode(gpu):
    # aion api/test_nn.zig:799-901: 2, (e^-3*2+3)/(e^-3+1), (e^-8*2+e^-4*3+4)/(e^-8+e^-4+1), abs 1e-4
    kc = np.zeros((1, 3, 1, 1), np.float32)
    vc = np.zeros((1, 3, 1, 1), np.float32)
    want = [2.0, (math.exp(-3) * 2 + 3) / (math.exp(-3) + 1),
            (math.exp(-8) * 2 + math.exp(-4) * 3 + 4) / (math.exp(-8) + math.exp(-4) + 1)]
    for t in range(3):
        kc[0, t, 0, 0] = vc[0, t, 0, 0] = t + 2
        q = np.full((1, 1, 1, 1), t + 2, np.float32)
        got = run_attention(gpu, q, kc, vc, 1.0, be.F32, be.F32, positions=np.array([[t]], np.int32), kv_lengths=np.array([t + 1], np.int32))
        assert abs(float(got.reshape(-1)[0]) - want[t]) < 1e-4


def test_generic_path_matches_oracle_on_odd_head_sizes(gpu, orc):
    rng = np.random.default_rng(3)
    q = rng.standard_normal((2, 9, 6, 40)).astype(np.float32)
    k = rng.standard_normal((2, 70, 3, 40)).astype(np.float32)
    v = rng.standard_normal((2, 70, 3, 24)).astype(np.float32)
    pos = np.tile(np.arange(61, 70, dtype=np.int32), (2, 1))
    got = run_attention(gpu, q, k, v, 0.2, be.F32, be.F32, positions=pos)
    ref = orc.attention_f64(q, k, v, 0.2, positions=pos)
    attn_err(got, ref, 1e-4)


def test_empty_window_and_plain_equals_cached(gpu, orc):
    (q, k, v, qd, kd), (qf, kf, vf) = make_qkv(17, 1, 33, 33, 8, 1, 64, "f16")
    zero = run_attention(gpu, q, k, v, 0.1, qd, kd, kv_lengths=np.array([0], np.int32))
    assert not zero.any()
    # plain sequence (implied positions / lengths) == explicit controls (aion cpu/test_cpu_backend.zig:1531)
    plain = run_attention(gpu, q, k, v, 0.1, qd, kd)
    cached = run_attention(gpu, q, k, v, 0.1, qd, kd, positions=np.arange(33, dtype=np.int32).reshape(1, 33), kv_lengths=np.array([33], np.int32))
    assert np.array_equal(plain, cached)


def test_attention_argument_errors(gpu):
    from aion_amd import hip
    a = gpu.alloc(1024)
    with pytest.raises(be.AionHipError) as e:
        gpu.step_attention(a, a, a, a, (1, 1, 4, 3, 2, 64, 64), 1.0)      # 3 q heads over 2 kv heads
    assert e.value.status == hip.INVALID_ARGUMENT
    with pytest.raises(be.AionHipError) as e:
        gpu.step_attention(a, a, a, a, (1, 1, 4, 2, 2, 64, 64), 1.0, kv_dtype=be.I32)
    assert e.value.status == hip.UNSUPPORTED
    a.free()


def test_precise_mode_brings_f32_queries_to_f32_accuracy(gpu, orc):
    (q, k, v, qd, kd), (qf, kf, vf) = make_qkv(23, 2, 1, 900, 8, 1, 256, "f16")
    pos = np.full((2, 1), 899, np.int32)
    ref = orc.attention_f64(qf, kf, vf, 1 / 16.0, positions=pos)
    fast = run_attention(gpu, q, k, v, 1 / 16.0, qd, kd, positions=pos)
    gpu.set_attention_precise(True)
    try:
        precise = run_attention(gpu, q, k, v, 1 / 16.0, qd, kd, positions=pos)
    finally:
        gpu.set_attention_precise(False)
    attn_err(fast, ref, 2e-3, "fast")
    e_prec = row_rms_err(precise, ref)
    say("  precise: worst row max|err|/rms(row)", e_prec)
    assert e_prec < 5e-5


def test_prefill_config4_sizes(gpu, orc):
    # BASELINE config 4a at L = 1024 and 2048: 8 q heads / 1 kv head, head size 256, bf16, scale 1/16, causal;
    # every row against the f64 reference (1e-2: bf16 MFMA operands). L = 512 is 32 prefill workgroups (an
    # eighth of the CUs: 16-row split kernel); L = 1024 and 2048 run on the prefill kernel with the key range of
    # every row tile cut into 4 and 2 segments that a merge pass folds. At L = 4096 the oracle is too slow for every row,
    # so the kernel is held to a sample of 30 positions over the whole range and to properties that do not depend on the size: V = const gives that const back (the
    # probabilities of a row sum to one), and row 0 sees key 0 only.
    for L, kernel in ((512, "attn_flash_split"), (1024, "attn_prefill"), (2048, "attn_prefill")):
        say("prefill config 4 L%d" % L)
        (q, k, v, qd, kd), (qf, kf, vf) = make_qkv(41, 1, L, L, 8, 1, 256, "bf16")
        got = run_attention(gpu, q, k, v, 1 / 16.0, qd, kd)
        assert gpu.last_kernel() == kernel
        ref = orc.attention_f64(qf, kf, vf, 1 / 16.0)
        attn_err(got, ref, 1e-2)
    say("prefill config 4 L4096 properties")
    L = 4096
    (q, k, v, qd, kd), (qf, kf, vf) = make_qkv(43, 1, L, L, 8, 1, 256, "bf16")
    ones, _ = to_bf16(np.full((1, L, 1, 256), 0.75, np.float32))
    got = run_attention(gpu, q, k, ones, 1 / 16.0, qd, kd)
    assert gpu.last_kernel() == "attn_prefill"
    assert row_rel_err(got, np.full_like(got, 0.75)) < 1e-2
    got = run_attention(gpu, q, k, v, 1 / 16.0, qd, kd)
    # one visible key: its value (the single probability is exp2 of a rounding residue, 1 to within an ulp)
    assert np.allclose(got[0, 0], np.broadcast_to(vf[0, 0, 0], (8, 256)), rtol=1e-6, atol=0)
    # the last rows against the reference on the last 16 positions only (full key range)
    ref_tail = orc.attention_f64(qf[:, L - 16:], kf, vf, 1 / 16.0, positions=np.arange(L - 16, L, dtype=np.int32).reshape(1, 16))
    attn_err(got[:, L - 16:], ref_tail, 1e-2)
    # and a sample of positions over the whole range against the reference: around the 128-row workgroup tiles (8 heads x 16
    # positions each), around the middle of the key range, where a row tile's two key segments meet, and in between
    idx = np.unique(np.array([1, 15, 16, 17, 63, 64, 200, 1000, 1023, 1024, 1025, 2040, 2047, 2048, 2049, 2111, 2112, 3000, 3071, 3072,
                              4000, 4079, 4080] + list(range(777, 4096, 512))))
    ref_s = orc.attention_f64(np.ascontiguousarray(qf[:, idx]), kf, vf, 1 / 16.0, positions=idx.astype(np.int32).reshape(1, -1))
    attn_err(got[:, idx], ref_s, 1e-2)
    # just past one workgroup per CU (260 row tiles on 256 CUs): two key segments per row tile again, because the longest
    # row tile alone would take as long as two average ones
    L = 4160
    say("prefill config 4 L4160 sample")
    (q, k, v, qd, kd), (qf, kf, vf) = make_qkv(47, 1, L, L, 8, 1, 256, "bf16")
    got = run_attention(gpu, q, k, v, 1 / 16.0, qd, kd)
    assert gpu.last_kernel() == "attn_prefill"
    idx = np.array([0, 1, 16, 1000, 2079, 2080, 2081, 3000, 4095, 4096, 4144, 4159])
    ref_s = orc.attention_f64(np.ascontiguousarray(qf[:, idx]), kf, vf, 1 / 16.0, positions=idx.astype(np.int32).reshape(1, -1))
    attn_err(got[:, idx], ref_s, 1e-2)


@pytest.mark.parametrize("B,Lq,T,lens,kernel", [
    (2, 96, 300, [256, 200], "attn_flash_split"),                 # 96 new rows at positions 160..255, capacity 300
    (4, 320, 520, [480, 400, 480, 170], "attn_prefill"),          # 320 new rows at positions 160..479, capacity 520
])
def test_prefill_chunk_with_positions_over_a_longer_cache(gpu, orc, B, Lq, T, lens, kernel):
    # a prompt chunk: new rows at positions 160.. over a longer cache; the sequences see different key counts
    Hq, Hkv, D = 8, 2, 128
    filled = 160 + Lq
    (q, k, v, qd, kd), (qf, kf, vf) = make_qkv(47, B, Lq, T, Hq, Hkv, D, "f16")
    k[:, filled:] = np.float16(np.nan)                   # beyond the cache length: must not leak
    v[:, filled:] = np.float16(np.nan)
    pos = np.tile(np.arange(160, filled, dtype=np.int32), (B, 1))
    lens = np.array(lens, np.int32)
    got = run_attention(gpu, q, k, v, 1 / math.sqrt(D), qd, kd, positions=pos, kv_lengths=lens)
    assert gpu.last_kernel() == kernel
    kz, vz = np.nan_to_num(kf), np.nan_to_num(vf)
    ref = orc.attention_f64(qf, kz, vz, 1 / math.sqrt(D), positions=pos, kv_lengths=lens)
    assert np.isfinite(got).all()
    attn_err(got, ref, 2e-3)


# A chunk of queries over a cache at least four times its length: with enough keys the 128-row kernel (keys cut into
# segments, partial results merged) takes over from the 16-row kernel well below the row count at which it takes a prompt
# over its own keys. 80 queries x 8 heads over 4096 keys at head size 256 -> 128-row kernel; 24 queries over the same cache
# stay on the 16-row kernel. The second sequence sees 1500 keys only (segments with nothing visible must contribute nothing).
@pytest.mark.parametrize("kind,tol", [("f16", 2e-3), ("bf16", 1e-2)])
@pytest.mark.parametrize("Lq,kernel", [(80, "attn_prefill"), (24, "attn_flash_split")])
def test_query_chunk_over_a_long_cache(gpu, orc, kind, tol, Lq, kernel):
    B, T, Hq, Hkv, D = 2, 4096, 8, 1, 256
    say("chunk over a long cache", kind, Lq)
    (q, k, v, qd, kd), (qf, kf, vf) = make_qkv(Lq, B, Lq, T, Hq, Hkv, D, kind)
    pos = np.tile(np.arange(T - Lq, T, dtype=np.int32), (B, 1))
    lens = np.array([T, 1500], np.int32)
    got = run_attention(gpu, q, k, v, 1 / math.sqrt(D), qd, kd, positions=pos, kv_lengths=lens)
    assert gpu.last_kernel() == kernel
    ref = orc.attention_f64(qf, kf, vf, 1 / math.sqrt(D), positions=pos, kv_lengths=lens)
    assert np.isfinite(got).all()
    attn_err(got, ref, tol)


def ring_of(linear, T):
    """The last T steps of a linear history [B, end, H, D], each at row t % T."""
    end = linear.shape[1]
    ring = np.zeros((linear.shape[0], T) + linear.shape[2:], linear.dtype)
    for t in range(max(0, end - T), end):
        ring[:, t % T] = linear[:, t]
    return ring


# Rolling caches (aion storage/cache.zig:202-207, cpu/exec/attention.zig:1072-1075, 1150-1152): the cache length
# exceeds the capacity, keys older than length - capacity are gone, key t is read from row t % capacity. Every
# kernel against the oracle's rolling attention (pinned to the linear one in tests/test_oracle_rolling.py).
@pytest.mark.parametrize("case", [
    # B, L, Hq, Hkv, D, T(capacity), ends, window, kind, kernel
    (2, 1, 8, 1, 256, 96, [250, 97], be.CAUSAL, "f16", "attn_flash_split"),            # decode, ring wrapped / barely wrapped
    (3, 1, 8, 2, 128, 2048, [5000, 2048, 700], (1000, 0, 0), "bf16", "attn_flash_split"),  # several segments, sliding window
    (2, 20, 4, 2, 64, 64, [300, 150], (30, 0, 0), "f16", "attn_flash_split"),          # a short chunk of new rows
    (4, 320, 8, 2, 128, 512, [1400, 900, 700, 330], (400, 0, 0), "f16", "attn_prefill"),   # long chunk: prefill kernel
    (2, 3, 4, 2, 80, 40, [130, 41], be.CAUSAL, "f16", "attn_generic"),                 # odd head size
    (2, 1, 8, 1, 64, 48, [200, 100], be.CAUSAL, "f16", "attn_generic"),                # ring shorter than a key tile
])
def test_rolling_caches(gpu, orc, case):
    B, L, Hq, Hkv, D, T, ends, window, kind, kernel = case
    say("rolling", case)
    rng = np.random.default_rng(sum(ends))
    ends = np.array(ends, np.int32)
    hist = int(ends.max())
    (q, k, v, qd, kd), (qf, kf, vf) = make_qkv(hist + L, B, L, hist, Hq, Hkv, D, kind)
    # every batch entry's ring holds ITS last T steps; queries sit at the end of each entry's history
    k_ring, v_ring = np.zeros((B, T, Hkv, D), k.dtype), np.zeros((B, T, Hkv, D), v.dtype)
    kr_f, vr_f = np.zeros((B, T, Hkv, D), np.float32), np.zeros((B, T, Hkv, D), np.float32)
    pos = np.zeros((B, L), np.int32)
    for b in range(B):
        e = int(ends[b])
        k_ring[b], v_ring[b] = ring_of(k[b:b + 1, :e], T)[0], ring_of(v[b:b + 1, :e], T)[0]
        kr_f[b], vr_f[b] = ring_of(kf[b:b + 1, :e], T)[0], ring_of(vf[b:b + 1, :e], T)[0]
        pos[b] = np.arange(e - L, e)
    got = run_attention(gpu, q, k_ring, v_ring, 1 / math.sqrt(D), qd, kd, window=window, positions=pos, kv_lengths=ends, rolling=True)
    assert gpu.last_kernel() == kernel
    want = orc.attention_rolling_f64(qf, kr_f, vr_f, 1 / math.sqrt(D), window, pos, ends)
    attn_err(got, want, (1e-2 if kind == "bf16" else 2e-3))


@pytest.mark.parametrize("window,rolling,soft_cap", [(be.CAUSAL, False, 0.0), ((300, 0, 0), False, 0.0), ((200, 40, 64), False, 0.0),
                                                     ((300, 0, 0), True, 0.0), (be.CAUSAL, False, 5.0)])
def test_prefill_key_segments_with_windows_and_ragged_lengths(gpu, orc, window, rolling, soft_cap):
    """The prefill kernel with its key range cut into segments (few row tiles on many CUs) and the merge pass: ragged
    cache lengths, positions that start inside the cache, windows that leave whole segments of a row tile empty, and
    a rolling cache. The profile must show the merge pass, or the case did not run in segments."""
    B, Lq, T, Hq, Hkv, D = 2, 400, 1536, 8, 2, 128
    ends = np.array([1500, 1000], np.int32)
    (q, k, v, qd, kd), (qf, kf, vf) = make_qkv(53, B, Lq, T, Hq, Hkv, D, "f16")
    pos = np.stack([np.arange(e - Lq, e, dtype=np.int32) for e in ends])
    if rolling:
        ends = ends + 2 * T                                   # the ring has wrapped twice
        pos = pos + 2 * T
    gpu.profile_start()
    got = run_attention(gpu, q, k, v, 1 / math.sqrt(D), qd, kd, window=window, positions=pos, kv_lengths=ends, rolling=rolling, soft_cap=soft_cap)
    names = [n for n, _ in gpu.profile_stop()]
    assert names == ["attn_prefill", "attn_merge"], names
    if rolling:
        ref = orc.attention_rolling_f64(qf, kf, vf, 1 / math.sqrt(D), window, pos, ends)
    else:
        ref = orc.attention_f64(qf, kf, vf, 1 / math.sqrt(D), window=window, soft_cap=soft_cap, positions=pos, kv_lengths=ends)
    assert np.isfinite(got).all()
    attn_err(got, ref, 2e-3)
