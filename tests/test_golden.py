"""The committed fixtures of tests/golden (written by tests/golden/make_golden.py: inputs of aion's
own tests, expected values agreed on by a numpy float64 restatement and the CPU oracle).

CPU tests hold the oracle to the fixtures; GPU tests hold the HIP path to them through the C ABI,
with no oracle in the loop. Bytes are compared bit-exactly; f32-accumulate results to the north-star
bound 2e-3 (floored, conftest.norm_err) plus 1e-5 of rms; attention to each case's stated tolerance.
"""
import json
import os

import numpy as np
import pytest

from conftest import norm_err, rms_err

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DT = {"q4_0": 3, "q8_0": 4}


def load(name):
    with open(os.path.join(GOLD, name + ".json")) as f:
        return json.load(f)


def f32(hexstr, shape=None):
    a = np.frombuffer(bytes.fromhex(hexstr), dtype="<f4").astype(np.float32)
    return a.reshape(shape) if shape is not None else a


def u8(hexstr):
    return np.frombuffer(bytes.fromhex(hexstr), dtype=np.uint8).copy()


# ---------------------------------------------------------------- CPU: oracle against fixtures
@pytest.mark.parametrize("case", load("quantize"), ids=lambda c: c["name"] + "-" + c["dtype"])
def test_oracle_quantizer_bytes(orc, case):
    vals = f32(case["values_f32_hex"], case["shape"])
    got = orc.quantize(DT[case["dtype"]], vals, case["quant_axis"]).reshape(-1)
    assert np.array_equal(got, u8(case["blocks_hex"]))


def oracle_matmul(orc, case, a, blocks, c_in):
    n, kw = case["n"], dict(alpha=case["alpha"], beta=case["beta"], c=c_in.copy())
    if case["weight"] == "q8_0 [N,K]":
        return orc.matmul_nt_q8(a, blocks, n, **kw)
    if case["weight"] == "q8_0 [K,N]":
        return orc.matmul_q8_kmajor(a, blocks, n, **kw)
    return orc.matmul_q_packed(3, a, blocks, n, **kw)


@pytest.mark.parametrize("case", load("matmul"), ids=lambda c: "%s-m%d-a%g" % (c["weight"], c["m"], c["alpha"]))
def test_oracle_matmul(orc, case):
    a = f32(case["a_f32_hex"], (case["m"], case["k"]))
    c_in = f32(case["c_in_f32_hex"], (case["m"], case["n"]))
    want = np.array(case["c_f64"]).reshape(case["m"], case["n"])
    got = oracle_matmul(orc, case, a, u8(case["blocks_hex"]), c_in)
    assert rms_err(got, want) < 1e-5


def test_oracle_attention(orc):
    for case in load("attention"):
        if "q" not in case:
            continue
        B, L, T, Hq, Hkv, Dk, Dv = case["shape"]
        q, k, v = f32(case["q"], (B, L, Hq, Dk)), f32(case["k"], (B, T, Hkv, Dk)), f32(case["v"], (B, T, Hkv, Dv))
        window = orc.CAUSAL if case["window"] is None else (case["window"][0], case["window"][1], 0)
        pos = np.array(case["positions"], np.int32).reshape(B, L)
        kl = np.array(case["kv_lengths"], np.int32)
        got = orc.attention_blocked(q, k, v, case["scale"], window=window, positions=pos, kv_lengths=kl)
        assert np.abs(got.reshape(-1) - np.array(case["out_f64"])).max() <= case["tol"]


def test_oracle_glue(orc):
    g = load("glue")
    x = f32(g["x_f32_hex"], (2, 16))
    gamma, beta = f32(g["gamma_f32_hex"]), f32(g["beta_f32_hex"])
    assert np.abs(orc.rmsnorm(x, gamma, g["eps"], beta=beta).reshape(-1) - np.array(g["rmsnorm_f64"])).max() < 1e-5
    assert np.abs(orc.gate_gelu(x * np.float32(g["gate_a_scale"]), x[::-1].copy()).reshape(-1) - np.array(g["gate_f64"])).max() < 2e-3
    pos = np.array([g["rope_positions"]], np.int32)
    assert np.abs(orc.rope(x.reshape(1, 2, 1, 16), pos, base=g["rope_base"]).reshape(-1) - np.array(g["rope_f64"])).max() < 1e-5
    assert orc.argmax(f32(g["argmax_in_f32_hex"], g["argmax_shape"])).tolist() == g["argmax"]


# ---------------------------------------------------------------- GPU: HIP path against fixtures
@pytest.mark.gpu
def test_gpu_quantizer_bytes(gpu):
    from aion_amd import backend as be
    for case in load("quantize"):
        vals = f32(case["values_f32_hex"], case["shape"])
        want = u8(case["blocks_hex"])
        host = be.quantize_blocks(DT[case["dtype"]], vals, case["quant_axis"]).reshape(-1)
        assert np.array_equal(host, want), ("host", case["name"], case["dtype"])
        src = gpu.upload(vals)
        dst = gpu.quantize_device(DT[case["dtype"]], src, case["shape"][0], case["shape"][1], case["quant_axis"])
        dev = gpu.download(dst, np.uint8, (want.size,))
        assert np.array_equal(dev, want), ("device", case["name"], case["dtype"])
        src.free(); dst.free()


@pytest.mark.gpu
def test_gpu_matmul(gpu):
    from aion_amd import backend as be
    for case in load("matmul"):
        m, n, k = case["m"], case["n"], case["k"]
        a = f32(case["a_f32_hex"], (m, k))
        c_in = f32(case["c_in_f32_hex"], (m, n))
        want = np.array(case["c_f64"]).reshape(m, n)
        dtype = be.Q8_0 if case["weight"].startswith("q8") else be.Q4_0
        layout = be.ROWS_NK if case["weight"].endswith("[N,K]") else be.KMAJOR_KN
        w = gpu.upload_weight(dtype, layout, n, k, u8(case["blocks_hex"]))
        got = gpu.matmul(w, a, alpha=case["alpha"], beta=case["beta"], c=c_in.copy())
        assert norm_err(got, want) < 2e-3 and rms_err(got, want) < 1e-5, (case["weight"], m, case["alpha"])
        w.free()


@pytest.mark.gpu
def test_gpu_attention(gpu):
    from aion_amd import backend as be
    from test_gpu_attention import run_attention
    for case in load("attention"):
        if "q" in case:
            B, L, T, Hq, Hkv, Dk, Dv = case["shape"]
            q, k, v = f32(case["q"], (B, L, Hq, Dk)), f32(case["k"], (B, T, Hkv, Dk)), f32(case["v"], (B, T, Hkv, Dv))
            window = be.CAUSAL if case["window"] is None else (case["window"][0], case["window"][1], 0)
            got = run_attention(gpu, q, k, v, case["scale"], be.F32, be.F32, window=window,
                                positions=np.array(case["positions"], np.int32).reshape(B, L),
                                kv_lengths=np.array(case["kv_lengths"], np.int32))
            assert np.abs(got.reshape(-1) - np.array(case["out_f64"])).max() <= case["tol"], case["name"]
        else:   # growing one-dim cache: step t appends k = v = values[t] and queries with it
            vals = case["values"]
            kc = np.zeros((1, len(vals), 1, 1), np.float32)
            for t, x in enumerate(vals):
                kc[0, t, 0, 0] = x
                got = run_attention(gpu, np.full((1, 1, 1, 1), x, np.float32), kc, kc.copy(), 1.0, be.F32, be.F32,
                                    positions=np.array([[t]], np.int32), kv_lengths=np.array([t + 1], np.int32))
                assert abs(float(got.reshape(-1)[0]) - case["out_f64"][t]) <= case["tol"]


@pytest.mark.gpu
def test_gpu_glue(gpu):
    g = load("glue")
    x = f32(g["x_f32_hex"], (2, 16))
    gamma, beta = f32(g["gamma_f32_hex"]), f32(g["beta_f32_hex"])
    dx, dg, db, out = gpu.upload(x), gpu.upload(gamma), gpu.upload(beta), gpu.alloc(2 * 16 * 4)
    gpu.step_rmsnorm(out, dx, dg, 2, 16, g["eps"], beta=db)
    assert np.abs(gpu.download(out, np.float32, (32,)) - np.array(g["rmsnorm_f64"])).max() < 1e-5
    da, dbb = gpu.upload(x * np.float32(g["gate_a_scale"])), gpu.upload(x[::-1].copy())
    gpu.step_gate_gelu(out, da, dbb, 32)
    assert np.abs(gpu.download(out, np.float32, (32,)) - np.array(g["gate_f64"])).max() < 2e-3
    pos = gpu.upload(np.array([g["rope_positions"]], np.int32))
    gpu.step_rope(out, dx, pos, 1, 2, 1, 16, base=g["rope_base"])
    assert np.abs(gpu.download(out, np.float32, (32,)) - np.array(g["rope_f64"])).max() < 1e-5
    am = f32(g["argmax_in_f32_hex"], g["argmax_shape"])
    dam, idx = gpu.upload(am), gpu.alloc(3 * 4)
    gpu.step_argmax(idx, dam, 3, 4)
    assert gpu.download(idx, np.int32, (3,)).tolist() == g["argmax"]
    for b in (dx, dg, db, out, da, dbb, pos, dam, idx):
        b.free()
