#!/usr/bin/env python3
"""Writes the small fixtures of this directory: python tests/golden/make_golden.py

Every expected value is computed here by a plain numpy restatement (float64 where the arithmetic is
floating point, exact integers otherwise) of the published aion formulas, on the deterministic inputs
of aion's own tests, and is then required to agree with the compiled CPU oracle before the file is
written: a fixture is a value two independent implementations agreed on. The fixtures are data only
(inputs and expected outputs as hex / numbers).

Inputs follow storage/quantize.zig:105-137 (vals[i] = ((i % 17) - 8) * 0.1 over [64,5], axis 0),
api/test_api.zig:4660-4700 (((i * 2654435761) % 2001 - 1000) * 0.001), cpu/kernels/matvec_q.zig:183-191
style index patterns for the activations, api/test_api.zig:3256-3331 and api/test_nn.zig:799-901 for
the attention known answers.
"""
import json
import math
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle as orc  # noqa: E402

Q4, Q8 = 3, 4


def hexf(a):
    return np.ascontiguousarray(a, dtype="<f4").tobytes().hex()


def rha(x):   # round half away from zero on exactly representable f64 input
    return np.sign(x) * np.floor(np.abs(x) + 0.5)


def q8_blocks(v):      # [nb,32] f32 -> [nb,34] u8
    v = v.astype(np.float32)
    amax = np.abs(v).max(axis=1)
    scale = np.where(amax == 0, np.float32(1), amax / np.float32(127)).astype(np.float32)
    s16 = scale.astype(np.float16)
    eff = s16.astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where((amax == 0) | (eff == 0), np.float32(0), np.float32(1) / eff).astype(np.float32)
    q = np.clip(rha((v * inv[:, None]).astype(np.float32).astype(np.float64)), -128, 127).astype(np.int8)
    out = np.zeros((v.shape[0], 34), np.uint8)
    out[:, :2] = s16.view(np.uint16).astype("<u2").view(np.uint8).reshape(-1, 2)
    out[:, 2:] = q.view(np.uint8)
    return out


def q4_blocks(v):      # [nb,32] f32 -> [nb,18] u8
    v = v.astype(np.float32)
    mx = np.abs(v).max(axis=1)
    scale = np.where(mx == 0, np.float32(1), mx / np.float32(7)).astype(np.float32)
    s16 = scale.astype(np.float16)
    q = np.clip(rha((v / scale[:, None]).astype(np.float32).astype(np.float64)), -8, 7).astype(np.int32) + 8
    out = np.zeros((v.shape[0], 18), np.uint8)
    out[:, :2] = s16.view(np.uint16).astype("<u2").view(np.uint8).reshape(-1, 2)
    out[:, 2:] = (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8)
    return out


def to_blocks(values, axis):
    """rank-2 f32 -> [nblocks,32] in the block order of the packed tensor (row-major over block space)."""
    r, c = values.shape
    if axis == 1:
        return values.reshape(r * (c // 32), 32)
    return values.reshape(r // 32, 32, c).transpose(0, 2, 1).reshape(-1, 32)


def decode(dtype, blocks):
    """[nb, 18|34] u8 -> (codes [nb,32] int, scale [nb] f64)"""
    s = blocks[:, :2].copy().view("<u2").view(np.float16).astype(np.float64).reshape(-1)
    if dtype == Q8:
        return blocks[:, 2:].view(np.int8).astype(np.int64), s
    b = blocks[:, 2:].astype(np.int64)
    codes = np.empty((blocks.shape[0], 32), np.int64)
    codes[:, 0::2] = (b & 15) - 8
    codes[:, 1::2] = (b >> 4) - 8
    return codes, s


def prepare_a(a):
    """activation rows -> (codes [m,kb,32] int, scale [m,kb] f32): cpu/kernels/matmul_q_i8.zig:187-203"""
    m, k = a.shape
    blk = a.astype(np.float32).reshape(m, k // 32, 32)
    amax = np.abs(blk).max(axis=2)
    with np.errstate(divide="ignore", invalid="ignore"):
        inv = np.where(amax == 0, np.float32(0), np.float32(127) / amax).astype(np.float32)
    q = np.clip(rha((blk * inv[:, :, None]).astype(np.float32).astype(np.float64)), -127, 127).astype(np.int64)
    scale = np.where(amax == 0, np.float32(0), amax / np.float32(127)).astype(np.float32)
    return q, scale


def quant_matmul(dtype, layout_nk, a, blocks, n, alpha, beta, c_in):
    """C = alpha * sum_kb f32(idot) * (a_s * w_s) + beta * C, summed in float64."""
    m, k = a.shape
    kb = k // 32
    codes, s = decode(dtype, blocks)
    if layout_nk:
        codes, s = codes.reshape(n, kb, 32), s.reshape(n, kb)
    else:
        codes, s = codes.reshape(kb, n, 32).transpose(1, 0, 2), s.reshape(kb, n).T
    aq, a_s = prepare_a(a)
    idot = np.einsum("mbi,nbi->mnb", aq, codes)
    f = (a_s.astype(np.float32)[:, None, :] * s.astype(np.float32)[None, :, :]).astype(np.float32).astype(np.float64)
    return alpha * (idot.astype(np.float64) * f).sum(axis=2) + beta * c_in.astype(np.float64)


def attention_f64(q, k, v, scale, left, right, positions, kv_lengths, soft_cap=0.0):
    b, l, hq, dk = q.shape
    t, hkv, dv = k.shape[1], k.shape[2], v.shape[3]
    out = np.zeros((b, l, hq, dv))
    for bi in range(b):
        for li in range(l):
            anchor = int(positions[bi, li])
            lo = 0 if left is None else anchor - min(anchor, left)
            hi = min(int(kv_lengths[bi]), anchor + 1 + right)
            for h in range(hq):
                g = h // (hq // hkv)
                if hi <= lo:
                    continue
                s = (k[bi, lo:hi, g].astype(np.float64) @ q[bi, li, h].astype(np.float64)) * scale
                if soft_cap > 0:
                    s = soft_cap * np.tanh(s / soft_cap)
                p = np.exp(s - s.max())
                out[bi, li, h] = (p[:, None] * v[bi, lo:hi, g].astype(np.float64)).sum(axis=0) / p.sum()
    return out


def main():
    gold = {}
    # ---- quantizer bytes
    qcases = []
    i = np.arange(64 * 5)
    pat_a = (((i % 17) - 8) * 0.1).astype(np.float32).reshape(64, 5)
    i = np.arange(4 * 96, dtype=np.uint64)
    pat_b = ((((i * 2654435761) % 2001).astype(np.int64) - 1000) * 0.001).astype(np.float32)
    special = np.zeros((4, 64), np.float32)
    special[0, :32] = 0.0                                                   # all-zero block
    special[0, 32:] = np.linspace(-1, 1, 32, dtype=np.float32)              # +-max at the ends
    special[1, :32] = np.array([(j - 16) * 0.5 for j in range(32)], np.float32)   # ties at x.5 after scaling
    special[1, 32:] = np.float32(65504.0) * np.linspace(-1, 1, 32, dtype=np.float32)
    special[2, :32] = np.float32(1e-8) * np.arange(32, dtype=np.float32)     # f16-subnormal scale
    special[2, 32:] = -np.arange(32, dtype=np.float32)
    special[3] = np.tile(np.array([127, -127, 63.5, -63.5, 7, -7, 3.5, -3.5], np.float32), 8)
    for name, vals, axis in (("mod17_64x5_axis0", pat_a, 0), ("knuth_4x96_axis1", pat_b.reshape(4, 96), 1),
                             ("knuth_96x4_axis0", pat_b.reshape(96, 4), 0), ("special_4x64_axis1", special, 1)):
        for dtype, fn, tag in ((Q8, q8_blocks, "q8_0"), (Q4, q4_blocks, "q4_0")):
            want = fn(to_blocks(vals, axis)).reshape(-1)
            got = orc.quantize(dtype, vals, axis).reshape(-1)
            assert np.array_equal(want, got), (name, tag)
            qcases.append({"name": name, "dtype": tag, "shape": list(vals.shape), "quant_axis": axis,
                           "values_f32_hex": hexf(vals), "blocks_hex": want.tobytes().hex()})
    gold["quantize"] = qcases

    # ---- small matmuls: q8 NT [8,64], q8 K-major [64,8], q4 K-major [64,8]; m = 1 and 3; alpha/beta
    mcases = []
    n, k = 8, 64
    j = np.arange(n * k)
    w = (np.sin(j * 0.37) * 0.05).astype(np.float32)
    for m in (1, 3):
        a = (np.cos(np.arange(m * k) * 0.11) * 1.5).astype(np.float32).reshape(m, k)
        a[0, 32:40] = 0.0
        c_in = (np.arange(m * n) * 0.25 - 1).astype(np.float32).reshape(m, n)
        for dtype, layout_nk, tag in ((Q8, True, "q8_0 [N,K]"), (Q8, False, "q8_0 [K,N]"), (Q4, False, "q4_0 [K,N]")):
            wv = w.reshape(n, k) if layout_nk else np.ascontiguousarray(w.reshape(n, k).T)
            blocks = orc.quantize(dtype, wv, 1 if layout_nk else 0)
            bb = blocks.reshape(-1, 34 if dtype == Q8 else 18)
            for alpha, beta in ((1.0, 0.0), (0.5, 2.0)):
                want = quant_matmul(dtype, layout_nk, a, bb, n, alpha, beta, c_in)
                if layout_nk:
                    got = orc.matmul_nt_q8(a, blocks, n, alpha=alpha, beta=beta, c=c_in.copy())
                elif dtype == Q8:
                    got = orc.matmul_q8_kmajor(a, blocks, n, alpha=alpha, beta=beta, c=c_in.copy())
                else:
                    got = orc.matmul_q_packed(dtype, a, blocks, n, alpha=alpha, beta=beta, c=c_in.copy())
                assert np.abs(got - want).max() <= 1e-6 * max(1.0, np.abs(want).max()), (tag, m, alpha)
                mcases.append({"weight": tag, "n": n, "k": k, "m": m, "alpha": alpha, "beta": beta,
                               "a_f32_hex": hexf(a), "c_in_f32_hex": hexf(c_in), "blocks_hex": blocks.reshape(-1).tobytes().hex(),
                               "c_f64": [float(x) for x in want.reshape(-1)]})
    gold["matmul"] = mcases

    # ---- attention: the two hand-computable aion cases and a 4-key GQA case
    acases = []
    q = np.zeros((1, 2, 4, 2), np.float32)
    kk = np.zeros((1, 6, 2, 2), np.float32)
    vv = np.zeros((1, 6, 2, 1), np.float32)
    for t in range(6):
        vv[0, t, 0, 0], vv[0, t, 1, 0] = t + 1, 10 * (t + 1)
    pos, kl = np.array([[4, 5]], np.int32), np.array([6], np.int32)
    want = attention_f64(q, kk, vv, 1.0, 2, 0, pos, kl)
    assert np.allclose(want.reshape(-1), [4, 4, 40, 40, 5, 5, 50, 50], atol=1e-12)
    acases.append({"name": "uniform_sliding_2_0", "q": hexf(q), "k": hexf(kk), "v": hexf(vv), "shape": [1, 2, 6, 4, 2, 2, 1],
                   "scale": 1.0, "window": [2, 0], "positions": pos.reshape(-1).tolist(), "kv_lengths": kl.tolist(),
                   "out_f64": want.reshape(-1).tolist(), "tol": 1e-6})
    rng = np.random.default_rng(20)
    q = rng.standard_normal((1, 2, 4, 8)).astype(np.float32)
    kk = rng.standard_normal((1, 4, 2, 8)).astype(np.float32)
    vv = rng.standard_normal((1, 4, 2, 8)).astype(np.float32)
    pos, kl = np.array([[2, 3]], np.int32), np.array([4], np.int32)
    want = attention_f64(q, kk, vv, 0.35, None, 0, pos, kl)
    got = orc.attention_f64(q, kk, vv, 0.35, positions=pos, kv_lengths=kl)
    assert np.abs(got - want).max() < 1e-6
    blocked = orc.attention_blocked(q, kk, vv, 0.35, positions=pos, kv_lengths=kl)
    assert np.abs(blocked - want).max() < 2e-4
    acases.append({"name": "causal_4key_gqa", "q": hexf(q), "k": hexf(kk), "v": hexf(vv), "shape": [1, 2, 4, 4, 2, 8, 8],
                   "scale": 0.35, "window": None, "positions": pos.reshape(-1).tolist(), "kv_lengths": kl.tolist(),
                   "out_f64": want.reshape(-1).tolist(), "tol": 2e-4})
    want3 = [2.0, (math.exp(-3) * 2 + 3) / (math.exp(-3) + 1),
             (math.exp(-8) * 2 + math.exp(-4) * 3 + 4) / (math.exp(-8) + math.exp(-4) + 1)]
    acases.append({"name": "three_step_decode", "values": [2.0, 3.0, 4.0], "out_f64": want3, "tol": 1e-4})
    gold["attention"] = acases

    # ---- glue: rmsnorm, gelu gate, rope (chunked halves), argmax (first maximum wins)
    x = (np.sin(np.arange(2 * 16) * 0.7) * 3).astype(np.float32).reshape(2, 16)
    gamma = (1 + 0.1 * np.arange(16)).astype(np.float32)
    beta = (0.01 * np.arange(16)).astype(np.float32)
    x64 = x.astype(np.float64)
    rn = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-6) * gamma + beta
    assert np.abs(orc.rmsnorm(x, gamma, 1e-6, beta=beta) - rn).max() < 1e-5
    g = x64 * 0.5
    gate = 0.5 * g * (1 + np.tanh(math.sqrt(2 / math.pi) * (g + 0.044715 * g ** 3))) * x64[::-1]
    assert np.abs(orc.gate_gelu((x * np.float32(0.5)), x[::-1].copy()) - gate).max() < 2e-3
    xr = x.reshape(1, 2, 1, 16)
    posr = np.array([[3, 17]], np.int32)
    half = 8
    freq = 10000.0 ** (-2.0 * np.arange(half) / 16)
    ang = posr.reshape(2, 1) * freq[None, :]
    rot = np.empty((2, 16))
    rot[:, :half] = x64[:, :half] * np.cos(ang) - x64[:, half:] * np.sin(ang)
    rot[:, half:] = x64[:, :half] * np.sin(ang) + x64[:, half:] * np.cos(ang)
    assert np.abs(orc.rope(xr, posr).reshape(2, 16) - rot).max() < 1e-5
    am = np.array([[1, 5, 5, -2], [7, 7, 7, 7], [-1, -3, -0.5, -0.5]], np.float32)
    assert orc.argmax(am).tolist() == [1, 0, 2]
    gold["glue"] = {"x_f32_hex": hexf(x), "gamma_f32_hex": hexf(gamma), "beta_f32_hex": hexf(beta), "eps": 1e-6,
                    "rmsnorm_f64": rn.reshape(-1).tolist(), "gate_a_scale": 0.5, "gate_f64": gate.reshape(-1).tolist(),
                    "rope_positions": [3, 17], "rope_base": 10000.0, "rope_f64": rot.reshape(-1).tolist(),
                    "argmax_in_f32_hex": hexf(am), "argmax_shape": [3, 4], "argmax": [1, 0, 2]}

    for name, obj in gold.items():
        path = os.path.join(HERE, name + ".json")
        with open(path, "w") as f:
            json.dump(obj, f, indent=0, separators=(",", ":"))
            f.write("\n")
        print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
