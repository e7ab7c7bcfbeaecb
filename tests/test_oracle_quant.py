"""Pins the oracle's quantizers and f16 conversion (CPU only).

Independent checks: numpy's IEEE float16 rounding, a vectorised numpy restatement evaluated
in float64 where that is exact, the inputs of the reference's own tests
(storage/quantize.zig:105-137, api/test_api.zig:4660-4700), and closed-form special cases.
"""
import numpy as np
import pytest


def round_half_away(x32):
    x = x32.astype(np.float64)           # exact widening; +0.5 is exact in f64 for |x| < 2^51
    return np.sign(x) * np.floor(np.abs(x) + 0.5)


def np_q8_blocks(vals_2d):
    """vals_2d: [nblocks, 32] f32 -> [nblocks, 34] u8, numpy restatement."""
    v = vals_2d.astype(np.float32)
    absmax = np.abs(v).max(axis=1)
    scale = np.where(absmax == 0, np.float32(1), absmax / np.float32(127)).astype(np.float32)
    s16 = scale.astype(np.float16)
    eff = s16.astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where((absmax == 0) | (eff == 0), np.float32(0), np.float32(1) / eff).astype(np.float32)
    prod = (v * inv[:, None]).astype(np.float32)
    q = np.clip(round_half_away(prod), -128, 127).astype(np.int8)
    out = np.zeros((v.shape[0], 34), dtype=np.uint8)
    out[:, 0:2] = s16.view(np.uint16)[:, None].view(np.uint8).reshape(-1, 2)
    out[:, 2:] = q.view(np.uint8)
    return out


def np_q4_blocks(vals_2d):
    v = vals_2d.astype(np.float32)
    mx = np.abs(v).max(axis=1)
    scale = np.where(mx == 0, np.float32(1), mx / np.float32(7)).astype(np.float32)
    s16 = scale.astype(np.float16)
    qf = (v / scale[:, None]).astype(np.float32)
    q = np.clip(round_half_away(qf), -8, 7).astype(np.int32) + 8
    out = np.zeros((v.shape[0], 18), dtype=np.uint8)
    out[:, 0:2] = s16.view(np.uint16)[:, None].view(np.uint8).reshape(-1, 2)
    out[:, 2:] = (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8)
    return out


def test_f16_roundtrip_all_halves(orc):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    for b in range(0, 65536, 7):
        got = orc.f16_bits_to_f32(b)
        w = want[b]
        if np.isnan(w):
            assert np.isnan(got)
        else:
            assert got == w
            assert orc.f32_to_f16_bits(w) == b


def test_f32_to_f16_matches_numpy_rne(orc):
    rng = np.random.default_rng(1)
    xs = np.concatenate([
        rng.standard_normal(4000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 5, 4000),
        # exact ties between neighbouring halves, and the overflow tie
        np.array([1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 65520.0, 65519.99, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                  2.0 ** -24 * 1.5, 2.0 ** -24 * 2.5, 6.1e-5, 0.0, -0.0, 70000.0, -70000.0], dtype=np.float32),
    ])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    for x, w in zip(xs, want):
        assert orc.f32_to_f16_bits(x) == int(w), (x, hex(int(w)))


def test_q8_reference_test_input_axis0(orc):
    # storage/quantize.zig:105-137: vals[i] = ((i % 17) - 8) * 0.1, shape [64, 5], axis 0
    K, N = 64, 5
    i = np.arange(K * N)
    vals = ((i % 17).astype(np.int32) - 8).astype(np.float32) * np.float32(0.1)
    got = orc.quantize(orc.Q8_0, vals.reshape(K, N), 0).reshape(K // 32, N, 34)
    blocks = vals.reshape(K // 32, 32, N).transpose(0, 2, 1).reshape(-1, 32)
    want = np_q8_blocks(blocks).reshape(K // 32, N, 34)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("dtype_name", ["q8", "q4"])
@pytest.mark.parametrize("shape,axis", [((64, 6), 0), ((6, 64), 1), ((3, 96, 4), 1), ((2, 3, 64), 2), ((128,), 0)])
def test_quantize_any_axis_matches_numpy(orc, dtype_name, shape, axis):
    # api/test_api.zig:4660-4700 input pattern
    n = int(np.prod(shape))
    i = np.arange(n, dtype=np.uint64)
    vals = (((i * np.uint64(2654435761)) % np.uint64(2001)).astype(np.int64) - 1000).astype(np.float32) * np.float32(0.001)
    v = vals.reshape(shape)
    dt = orc.Q8_0 if dtype_name == "q8" else orc.Q4_0
    got = orc.quantize(dt, v, axis)
    moved = np.moveaxis(v, axis, -1)                       # [..., axis]
    lead = moved.shape[:-1]
    blocks = moved.reshape(lead + (shape[axis] // 32, 32))
    blocks = np.moveaxis(blocks, -2, axis)                 # block index back in the axis position
    flat = np.ascontiguousarray(blocks).reshape(-1, 32)
    want = (np_q8_blocks if dtype_name == "q8" else np_q4_blocks)(flat)
    assert np.array_equal(got.reshape(want.shape), want)
    # same bytes from a transposed layout: [K,N] axis 0 is a block permutation of [N,K] axis 1
    if len(shape) == 2 and axis == 0:
        K, N = shape
        bb = orc.BLOCK_BYTES[dt]
        t = orc.quantize(dt, np.ascontiguousarray(v.T), 1).reshape(N, K // 32, bb)
        assert np.array_equal(got.reshape(K // 32, N, bb), t.transpose(1, 0, 2))


def test_quantize_special_cases(orc):
    z = np.zeros((1, 32), np.float32)
    b = orc.quantize(orc.Q8_0, z, 1)
    assert b[0] == 0x00 and b[1] == 0x3C and not b[2:].any()          # f16(1.0) = 0x3C00, zero codes
    b4 = orc.quantize(orc.Q4_0, z, 1)
    assert b4[0] == 0x00 and b4[1] == 0x3C and (b4[2:] == 0x88).all()  # code 0 -> nibble 8
    v = np.zeros((1, 32), np.float32)
    v[0, 0], v[0, 1], v[0, 2] = 2.54, -2.54, 1.27
    b = orc.quantize(orc.Q8_0, v, 1)
    q = b[2:].view(np.int8)
    assert q[0] == 127 and q[1] == -127
    s = np.array([int(b[0]) | (int(b[1]) << 8)], np.uint16).view(np.float16).astype(np.float32)[0]
    assert q[2] == int(np.sign(1.27) * np.floor(abs(np.float32(1.27) * (np.float32(1) / s)) + 0.5))
    b4 = orc.quantize(orc.Q4_0, v, 1)
    assert (b4[2] & 15) == 15 and (b4[2] >> 4) == 1                     # +7 -> 15 low nibble, -7 -> 1 high nibble
    # half-away-from-zero ties: scale exactly 1.0 (absmax 127 / 7) so v/scale is exact
    v = np.zeros((1, 32), np.float32)
    v[0, :6] = [127, 0.5, -0.5, 1.5, 2.5, -2.5]
    q = orc.quantize(orc.Q8_0, v, 1)[2:].view(np.int8)
    assert list(q[:6]) == [127, 1, -1, 2, 3, -3]
    v[0, 0] = 7
    nb = orc.quantize(orc.Q4_0, v, 1)[2:]
    codes = np.stack([nb & 15, nb >> 4], 1).reshape(-1).astype(int) - 8
    assert list(codes[:6]) == [7, 1, -1, 2, 3, -3]


def test_q4_divides_by_the_unrounded_scale_hand_computed_block(orc):
    # aion cpu/test_cpu_kernels.zig:490-523: q = round(v / scale) with scale = max_abs / 7 in f32, while the STORED scale is
    # f16(scale). Block: max_abs = 7 * (1 + 2^-12), so scale = 1 + 2^-12 exactly and f16(scale) = 1.0 (half an f16 ulp at 1 is
    # 2^-11). Then 2.5 / scale = 2.4994 -> 2, -2.5 -> -2, 0.5 / scale = 0.49988 -> 0; a quantizer that divided by the
    # stored (rounded) scale would hit the exact ties 2.5, -2.5, 0.5 and give 3, -3, 1.
    v = np.zeros((1, 32), np.float32)
    v[0, :4] = [7.0 + 7.0 / 4096.0, 2.5, -2.5, 0.5]
    assert float(v[0, 0]) == 7.0 + 7.0 / 4096.0 and np.float32(v[0, 0]) / np.float32(7) == np.float32(1 + 2.0 ** -12)
    b = orc.quantize(orc.Q4_0, v, 1)
    want = bytes([0x00, 0x3C,                     # f16(1.000244) = 1.0
                  (7 + 8) | ((2 + 8) << 4),       # elements 0 (low nibble) and 1 (high nibble)
                  (-2 + 8) | ((0 + 8) << 4)]      # elements 2 and 3
                 + [0x88] * 14)
    assert b.tobytes() == want
    # the same block through the q8_0 quantizer, which DOES divide by the f16-rounded scale (storage/quantize.zig:83-103):
    # absmax / 127 = 0.055131567 -> f16 0.055145264; 2.5 / that = 45.335 -> 45 either way, so pin it with the stored bits
    b8 = orc.quantize(orc.Q8_0, v, 1)
    s16 = np.array([np.float32(v[0, 0]) / np.float32(127)], np.float32).astype(np.float16)
    assert b8[:2].tobytes() == s16.tobytes() and b8[2:3].view(np.int8)[0] == 127


def test_quantize_rejects_bad_axis(orc):
    with pytest.raises(ValueError):
        orc.quantize(orc.Q8_0, np.zeros((33, 4), np.float32), 0)


@pytest.mark.parametrize("dt_name", ["q8", "q4"])
def test_dequantize_is_code_times_scale(orc, dt_name):
    rng = np.random.default_rng(5)
    dt = orc.Q8_0 if dt_name == "q8" else orc.Q4_0
    w = (rng.standard_normal((64, 8)) * 0.02).astype(np.float32)
    blk = orc.quantize(dt, w, 0)
    deq = orc.dequantize(dt, blk, (64, 8), 0)
    step = np.abs(w).reshape(2, 32, 8).max(axis=1) / (127 if dt_name == "q8" else 7)
    err = np.abs(deq - w).reshape(2, 32, 8).max(axis=1)
    assert (err <= step * 0.51 + 1e-6).all()   # q4 may clamp +7.5 -> 7: covered by the 0.51 step bound on |v|<=max
