"""Pins the oracle's rolling-cache attention and append (oracle.attention_rolling_f64, oracle.sequence_append) to the
already pinned linear attention (orc_attention_f64): a ring is a linear cache seen through t -> t % T, so
  (1) while every query's window stays inside the retained keys, ring == linear over the whole history;
  (2) when the window reaches further back than the ring holds, ring == the linear cache with the overwritten
      prefix cut off and every position shifted down by the cut (exact for windows without chunking);
  (3) appending step by step into a ring and reading rows back by t % T returns the last T steps."""
import numpy as np
import pytest

from oracle import oracle as orc


def ring_of(linear, T):
    end = linear.shape[1]
    ring = np.full((linear.shape[0], T) + linear.shape[2:], np.nan, linear.dtype)
    for t in range(max(0, end - T), end):
        ring[:, t % T] = linear[:, t]
    return np.nan_to_num(ring)


@pytest.mark.parametrize("window", [(40, 0, 0), (24, 3, 0), (16, 0, 8)])
def test_ring_equals_linear_while_the_window_stays_inside_the_ring(window):
    rng = np.random.default_rng(1)
    B, L, Hq, Hkv, D, T, end = 2, 6, 4, 2, 16, 64, 150
    q = rng.standard_normal((B, L, Hq, D)).astype(np.float32)
    k = rng.standard_normal((B, end, Hkv, D)).astype(np.float32)
    v = rng.standard_normal((B, end, Hkv, D)).astype(np.float32)
    pos = np.tile(np.arange(end - L, end, dtype=np.int32), (B, 1))
    lens = np.full(B, end, np.int32)
    want = orc.attention_f64(q, k, v, 0.25, window=window, positions=pos, kv_lengths=lens)
    got = orc.attention_rolling_f64(q, ring_of(k, T), ring_of(v, T), 0.25, window, pos, lens)
    assert np.abs(got - want).max() < 1e-5


def test_ring_drops_what_was_overwritten():
    rng = np.random.default_rng(2)
    B, L, Hq, Hkv, D, T = 2, 5, 4, 1, 8, 32
    ends = np.array([90, 41], np.int32)
    q = rng.standard_normal((B, L, Hq, D)).astype(np.float32)
    got_all, want_all = [], []
    for b in range(B):
        end, cut = int(ends[b]), int(ends[b]) - T
        k = rng.standard_normal((1, end, Hkv, D)).astype(np.float32)
        v = rng.standard_normal((1, end, Hkv, D)).astype(np.float32)
        pos = np.arange(end - L, end, dtype=np.int32).reshape(1, L)
        got_all.append(orc.attention_rolling_f64(q[b:b + 1], ring_of(k, T), ring_of(v, T), 0.3, orc.CAUSAL, pos, ends[b:b + 1]))
        want_all.append(orc.attention_f64(q[b:b + 1], k[:, cut:], v[:, cut:], 0.3, window=orc.CAUSAL, positions=pos - cut,
                                          kv_lengths=np.array([T], np.int32)))
    assert np.abs(np.concatenate(got_all) - np.concatenate(want_all)).max() < 1e-5


def test_append_into_a_ring_keeps_the_last_steps():
    rng = np.random.default_rng(3)
    B, T, H, D = 2, 8, 2, 4
    cache = np.zeros((B, T, H, D), np.float16)
    history = rng.standard_normal((B, 21, H, D)).astype(np.float16)
    t = 0
    for n in (3, 5, 1, 8, 4):
        cache = orc.sequence_append(cache, history[:, t:t + n], np.array([t, t], np.int32), rolling=True)
        t += n
    for step in range(t - T, t):
        assert np.array_equal(cache[:, step % T], history[:, step])
    with pytest.raises(ValueError):
        orc.sequence_append(np.zeros((B, T, H, D), np.float16), history[:, :3], np.array([6, 0], np.int32))
    # one write index per batch entry (sequence_append.zig:58-60)
    lin = orc.sequence_append(np.zeros((B, T, H, D), np.float16), history[:, :2], np.array([1, 5], np.int32))
    assert np.array_equal(lin[0, 1:3], history[0, :2]) and np.array_equal(lin[1, 5:7], history[1, :2])
    assert not lin[0, 5:7].any() and not lin[1, 1:3].any()
