"""Pins the oracle's cache-growth restatements (oracle.grow_target, grow_axis, grow_rolling, session_growth_target) to
the reference's own known answers:
  - storage/test_storage.zig:883-898  a ring [4,5,0,3] (capacity 4, end 6, 3 retained) grown to 7 -> [0,0,0,3,4,5,0];
  - backend/cpu/test_cpu_backend.zig:4718-4790  a growable cache [0,1,2,3] appended [90,91] at 5 -> capacity 8,
    [0,1,2,3,0,90,91,0];
  - storage/test_storage.zig:862-873  capacity 8 with factor 2/1 asked for step 8 -> 16;
  - api/test_api_gpu.zig:219-283  initial 2, factor 2/1, ceiling 8, five one-row appends -> [1,2,3,4,5,0,0,0];
  - api/loaded_model.zig:808-817  "bounds a 32 -> 2048 session to three shapes";
and to what the definitions fix: a grown ring read through t % capacity returns exactly the retained steps."""
import numpy as np
import pytest

from oracle import oracle as orc


def test_rolling_growth_golden_vector():
    ring = np.array([4, 5, 0, 3], np.float32).reshape(1, 4, 1, 1)
    got = orc.grow_rolling(ring, 7, 3, [6])
    assert got.reshape(-1).tolist() == [0, 0, 0, 3, 4, 5, 0]


def test_growable_append_golden_vector():
    cache = np.array([0, 1, 2, 3], np.float32).reshape(1, 4, 1, 1)
    new = np.array([90, 91], np.float32).reshape(1, 2, 1, 1)
    # store_view.zig:104-124: grow while target <= the step being mapped (here up to step 6)
    target = 4
    while target <= 6:
        target = orc.grow_target(target, 2, 1)
    assert target == 8
    grown = orc.grow_axis(cache, 1, target)
    out = orc.sequence_append(grown, new, np.array([5], np.int32))
    assert out.reshape(-1).tolist() == [0, 1, 2, 3, 0, 90, 91, 0]


def test_growth_schedule():
    assert orc.grow_target(8, 2, 1) == 16
    assert orc.grow_target(2, 3, 2) == 3          # ceil(2 * 3 / 2)
    assert orc.grow_target(3, 3, 2) == 5          # ceil(4.5)
    assert orc.grow_target(5, 1, 1) == 6          # no growth by the factor: one more row
    assert orc.grow_target(7, 1, 2) == 8
    for bad in ((0, 2, 1), (4, 0, 1), (4, 2, 0)):
        with pytest.raises(ValueError):
            orc.grow_target(*bad)


def test_session_growth_is_quantized():
    # a 32 -> 2048 token-at-a-time session sees three capacities
    caps, cap = [32], 32
    for pos in range(2048):
        if pos + 1 > cap:
            cap = orc.session_growth_target(cap, pos + 1, 3, 2)
            caps.append(cap)
    assert caps == [32, 128, 512, 2048]
    assert orc.session_growth_target(2, 3, 2, 1, max_capacity=8) == 8      # 4x the old capacity, clipped to the ceiling
    assert orc.session_growth_target(100, 101, 2, 1) == 400               # at least four times
    assert orc.session_growth_target(100, 900, 2, 1) == 2048              # 100 -> 200 -> 400 -> 800 -> 1600, then the power of two above
    with pytest.raises(ValueError):
        orc.session_growth_target(4, 9, 2, 1, max_capacity=8)


def test_five_appends_into_a_growing_cache():
    # the api test's session on the oracle: capacity 2, factor 2/1, ceiling 8, one row per run
    cache = np.zeros((1, 2, 1, 1), np.float32)
    for pos in range(5):
        if pos + 1 > cache.shape[1]:
            cache = orc.grow_axis(cache, 1, orc.session_growth_target(cache.shape[1], pos + 1, 2, 1, max_capacity=8))
        cache = orc.sequence_append(cache, np.full((1, 1, 1, 1), pos + 1, np.float32), np.array([pos], np.int32))
    assert cache.reshape(-1).tolist() == [1, 2, 3, 4, 5, 0, 0, 0]


@pytest.mark.parametrize("T,new_T,retained,ends", [(8, 32, 5, [3, 40]), (16, 17, 16, [16, 100]), (4, 64, 100, [0, 7]), (6, 13, 1, [5, 6])])
def test_grown_ring_holds_exactly_the_retained_steps(T, new_T, retained, ends):
    rng = np.random.default_rng(5)
    B, H, D = len(ends), 2, 3
    hist = rng.standard_normal((B, max(ends) + 1, H, D)).astype(np.float32) + 10.0     # no zeros
    ring = np.zeros((B, T, H, D), np.float32)
    for b, end in enumerate(ends):
        for t in range(max(0, end - T), end):
            ring[b, t % T] = hist[b, t]
    grown = orc.grow_rolling(ring, new_T, retained, ends)
    assert grown.shape == (B, new_T, H, D)
    for b, end in enumerate(ends):
        kept = min(end, retained, T)
        rows = set()
        for t in range(end - kept, end):
            assert np.array_equal(grown[b, t % new_T], hist[b, t])
            rows.add(t % new_T)
        for p in set(range(new_T)) - rows:
            assert not grown[b, p].any()


def test_grow_axis_keeps_indices():
    rng = np.random.default_rng(6)
    x = rng.standard_normal((3, 5, 2, 4)).astype(np.float16)
    y = orc.grow_axis(x, 1, 9)
    assert y.shape == (3, 9, 2, 4) and np.array_equal(y[:, :5], x) and not y[:, 5:].any()
    assert np.array_equal(orc.grow_axis(x, 1, 5), x)
    with pytest.raises(ValueError):
        orc.grow_axis(x, 1, 4)
