"""Pins the node-by-node graph interpreter (oracle/graph_oracle.py) to the hand-written C++ oracle decoder
(oracle/aion_oracle.cpp orc_decoder_forward, itself pinned step by step elsewhere): the plain decoder package holds
the same computation as that decoder, so the two must give the same logits bit for bit - same restated steps, same
order of operations (the gate is Unary(gelu) then multiply on one side and the fused gate on the other: bit-identical
by cpu/exec/elementwise.zig:25-37). Also the elementwise restatements against closed forms."""
import numpy as np
import pytest

from aion_amd import aion_file
from oracle import aion_writer, graph_oracle
from oracle import oracle as orc

CFG = dict(layers=2, hidden=64, heads=4, kv_heads=2, head_dim=32, ffn=96, vocab=64, eps=1e-6, rope_base=10000.0)
SHAPES = {"wq": (64, 128), "wk": (64, 64), "wv": (64, 64), "wo": (128, 64), "wgate": (64, 96), "wup": (64, 96), "wdown": (96, 64)}


def weights(wdtype, seed=3):
    rng = np.random.default_rng(seed)
    dt = orc.Q4_0 if wdtype == "q4_0" else orc.Q8_0
    blocks = {}
    names = ["l%d.%s" % (l, n) for l in range(CFG["layers"]) for n in SHAPES] + ["lm_head"]
    for name in names:
        k, n = SHAPES.get(name.split(".")[-1], (CFG["hidden"], CFG["vocab"]))
        w = (rng.standard_normal((k, n)) * 0.08).astype(np.float32)
        # q4: [K,N] blocks along K (quant_axis 0); q8: [N,K] rows (quant_axis 1), used through a transpose
        blocks[name] = orc.quantize(dt, w, 0) if wdtype == "q4_0" else orc.quantize(dt, np.ascontiguousarray(w.T), 1)
    embed = rng.standard_normal((CFG["vocab"], CFG["hidden"])).astype(np.float32)
    gammas = {"l%d.norm%d" % (l, i): (1 + 0.1 * rng.standard_normal(CFG["hidden"])).astype(np.float32) for l in range(CFG["layers"]) for i in (1, 2)}
    gammas["norm_f"] = (1 + 0.1 * rng.standard_normal(CFG["hidden"])).astype(np.float32)
    return blocks, embed, gammas


@pytest.mark.parametrize("wdtype", ["q4_0", "q8_0"])
def test_interpreter_equals_the_oracle_decoder(wdtype):
    blocks, embed, gammas = weights(wdtype)
    cfg = dict(CFG, wdtype=wdtype)
    pkg = aion_file.parse(aion_writer.build_decoder_package(cfg, lambda name: blocks[name], embed, gammas=gammas))
    T = 24
    dec = orc.Decoder(cfg["layers"], cfg["hidden"], cfg["heads"], cfg["kv_heads"], cfg["head_dim"], cfg["ffn"], cfg["vocab"], T,
                      eps=cfg["eps"], rope_base=cfg["rope_base"], wdtype=orc.Q4_0 if wdtype == "q4_0" else orc.Q8_0, threads=2)
    for name, b in blocks.items():
        dec.set_weight(name, b)
    dec.set_weight("embed", embed)
    for name, g in gammas.items():
        dec.set_weight(name, g)
    caches = {name: np.zeros((1, T, cfg["kv_heads"], cfg["head_dim"]), np.float16) for name, _ in pkg.inputs if name.endswith("_cache")}
    rng = np.random.default_rng(7)
    pos = 0
    for s in (6, 1, 1, 3):
        tokens = rng.integers(0, cfg["vocab"], s).astype(np.int32)
        feeds = dict(caches)
        by_role = {"tokens": tokens.reshape(1, s), "positions": np.arange(pos, pos + s, dtype=np.int32).reshape(1, s),
                   "cache_write_index": np.array([pos], np.int32), "cache_visible_end": np.array([pos + s], np.int32)}
        for idx, (name, _vid) in enumerate(pkg.inputs):
            role = pkg.role_of_input(idx)
            if role.kind in by_role:
                feeds[name] = by_role[role.kind]
        out = graph_oracle.run_graph(pkg, feeds, {"seq": s, "ctx": T})
        tok, logits = dec.forward(tokens, pos)
        assert np.array_equal(out["logits"][0, -1], logits)
        assert int(out["next_token"][0, -1]) == tok
        for name in caches:
            caches[name] = out[name]
        pos += s


def test_elementwise_restatements():
    x = np.linspace(-9, 9, 73).astype(np.float32)
    # sigmoid and tanh are aion's exp-polynomial approximations: close to the functions, not equal to them
    assert np.abs(orc.unary("sigmoid", x) - 1 / (1 + np.exp(-x.astype(np.float64)))).max() < 2e-5
    assert np.abs(orc.unary("tanh", x) - np.tanh(x.astype(np.float64))).max() < 4e-5
    assert np.array_equal(orc.unary("tanh", x), np.array([orc.tanh_approx(float(v)) for v in x], np.float32))
    assert np.array_equal(orc.unary("relu", x), np.maximum(x, 0))
    assert np.array_equal(orc.unary("silu", x), x * orc.unary("sigmoid", x))
    assert np.array_equal(orc.unary("sqrt", np.abs(x)), np.sqrt(np.abs(x)))
    # Unary(gelu) then multiply == the fused gate, bit for bit (cpu/exec/elementwise.zig:25-37)
    up = np.cos(x).astype(np.float32)
    assert np.array_equal(orc.binary("mul", orc.unary("gelu", x), up), orc.gate_gelu(x, up))
    a = np.arange(24, dtype=np.float32).reshape(2, 3, 4) - 7
    for op, f in (("add", np.add), ("sub", np.subtract), ("mul", np.multiply), ("div", np.divide)):
        for b in (a[::-1].copy() + 0.5, np.array([3.0], np.float32), np.array([1, 2, 4, 8], np.float32), (np.arange(12, dtype=np.float32) + 1).reshape(3, 4)):
            assert np.array_equal(orc.binary(op, a, b), f(a, b).astype(np.float32)), (op, b.shape)
    with pytest.raises(ValueError):
        orc.binary("add", a, np.ones(5, np.float32))
