"""A decoder `.aion` package (made by oracle/aion_writer.py) run through aion_amd/package.py on the GPU, against the
CPU oracle decoder fed the same weights, teacher-forced, with the tolerance of tests/test_gpu_decoder.py (the GPU
must be no further from the oracle than the oracle's own sensitivity to the exp it uses in attention); and against
the fused step sequence of aion_amd/decoder.py, which must pick the same tokens from the same weights."""
import sys

import numpy as np
import pytest

from aion_amd import aion_file, backend as be
from aion_amd.decoder import Decoder, DecoderConfig, SyntheticWeights, weight_shapes
from aion_amd.package import PackageRunner, Unsupported
from oracle import aion_writer

pytestmark = pytest.mark.gpu

SMALL = dict(layers=3, hidden=512, heads=8, kv_heads=1, head_dim=64, ffn=1024, vocab=2048, max_seq=48)


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def package_bytes(cfg, weights):
    d = dict(layers=cfg.layers, hidden=cfg.hidden, heads=cfg.heads, kv_heads=cfg.kv_heads, head_dim=cfg.head_dim, ffn=cfg.ffn,
             vocab=cfg.vocab, eps=cfg.eps, rope_base=cfg.rope_base, wdtype="q8_0" if cfg.wdtype == be.Q8_0 else "q4_0")
    return aion_writer.build_decoder_package(d, weights.blocks, weights.embed())


@pytest.mark.parametrize("wdtype", [be.Q4_0, be.Q8_0])
def test_package_runs_like_the_oracle_decoder(gpu, orc, wdtype):
    cfg = DecoderConfig(wdtype=wdtype, **SMALL)
    weights = SyntheticWeights(cfg, 5)
    pkg = aion_file.parse(package_bytes(cfg, weights))
    mk = lambda exact: orc.Decoder(cfg.layers, cfg.hidden, cfg.heads, cfg.kv_heads, cfg.head_dim, cfg.ffn, cfg.vocab, cfg.max_seq,
                                   eps=cfg.eps, rope_base=cfg.rope_base, wdtype=cfg.wdtype, threads=8, attn_exact=exact)
    ref, alt = mk(False), mk(True)
    ones = np.ones(cfg.hidden, np.float32)
    for o in (ref, alt):
        for name in weight_shapes(cfg):
            o.set_weight(name, weights.blocks(name))
        o.set_weight("embed", weights.embed())
        for l in range(cfg.layers):
            o.set_weight("l%d.norm1" % l, ones)
            o.set_weight("l%d.norm2" % l, ones)
        o.set_weight("norm_f", ones)
    run = PackageRunner(gpu, pkg, capacity=cfg.max_seq)
    fused = Decoder(gpu, cfg, weights)
    try:
        prompt = np.random.default_rng(9).integers(0, cfg.vocab, 16).astype(np.int32)
        errs, selfs = [], []

        def step(tokens, pos):
            out = run.run(tokens, want=("next_token", "logits"))
            logits, tok = out["logits"][0, -1], int(out["next_token"][0, -1])
            (otok, ologits), (_, alogits) = ref.forward(tokens, pos), alt.forward(tokens, pos)
            rms = float(np.sqrt((ologits.astype(np.float64) ** 2).mean()))
            err, self_err = float(np.abs(logits - ologits).max()) / rms, float(np.abs(alogits - ologits).max()) / rms
            top2 = np.sort(ologits)[-2:]
            say("  pos %d: package max|err|/rms %.2e, cpu self-sensitivity %.2e, tokens %d / %d" % (pos, err, self_err, tok, otok))
            if float(top2[1] - top2[0]) / rms > 2 * err:
                assert tok == otok
            errs.append(err); selfs.append(self_err)
            return tok, logits

        tok, logits = step(prompt, 0)
        ftok = fused.prefill(prompt)
        flogits = fused.logits_host()
        # the fused step sequence sees the same weights: same arithmetic up to summation order
        assert float(np.abs(flogits - logits).max()) <= 3 * max(selfs) * float(np.sqrt((logits.astype(np.float64) ** 2).mean())) + 1e-3
        pos = prompt.size
        for _ in range(6):
            tok, _ = step(np.array([tok], np.int32), pos)
            pos += 1
        assert run.pos == pos
        assert np.mean(errs) < 2 * np.mean(selfs) + 1e-3 and max(errs) < 3 * max(selfs) + 1e-3
    finally:
        run.close(); fused.close()


def test_package_runner_refuses_what_the_backend_has_no_step_for(gpu):
    b = aion_writer.PackageBuilder()
    seq = b.symbol("seq")
    x = b.input("tokens", "i32", (1, seq), role="tokens", axis=1)
    table = b.initializer("f32", (8, 32), b.tensor_plain("f32", np.zeros((8, 32), np.float32)), "embed")
    e = b.gather(table, x, (1, seq, 32))
    y = b.unary("log", b.unary("tanh", e, (1, seq, 32)), (1, seq, 32))        # tanh has a step, log has none
    b.output("y", y)
    pkg = aion_file.parse(b.to_bytes())
    run = PackageRunner(gpu, pkg, capacity=8)
    try:
        with pytest.raises(Unsupported):
            run.run(np.array([1, 2], np.int32), want=("y",))
    finally:
        run.close()


def test_package_with_an_f32_head_runs_as_matmul_nt(gpu, orc):
    """MatMul over the ViewTranspose2D of a plain f32 [N,K] initializer is MatMulNT with an f32 B (graph/program/compiler.zig:
    337-357): tokens -> f32 embedding rows -> RMSNorm -> the f32 head, for one and for several tokens, against the node-by-node
    interpreter. Nothing on this path is quantized, so the bar is the f32 one (1e-5 of the logits' rms)."""
    from oracle import graph_oracle
    V, E, N = 64, 96, 200
    rng = np.random.default_rng(31)
    b = aion_writer.PackageBuilder()
    seq = b.symbol("seq")
    x = b.input("tokens", "i32", (1, seq), role="tokens", axis=1)
    table = b.initializer("f32", (V, E), b.tensor_plain("f32", rng.standard_normal((V, E)).astype(np.float32)), "embed")
    gamma = b.initializer("f32", (E,), b.tensor_plain("f32", (1 + 0.1 * rng.standard_normal(E)).astype(np.float32)), "gamma")
    beta = b.initializer("f32", (E,), b.tensor_plain("f32", np.zeros(E, np.float32)), "beta")
    head = b.initializer("f32", (N, E), b.tensor_plain("f32", (rng.standard_normal((N, E)) * 0.1).astype(np.float32)), "head")
    h = b.rmsnorm(b.gather(table, x, (1, seq, E)), gamma, beta, 1e-6, (1, seq, E), (E,))
    logits = b.matmul(h, b.transpose2d(head, "f32", (E, N)), (1, seq, N), alpha=0.5)
    b.output("logits", logits)
    pkg = aion_file.parse(b.to_bytes())
    run = PackageRunner(gpu, pkg, capacity=8)
    try:
        for tokens in (np.array([5], np.int32), np.array([1, 63, 7, 7, 0], np.int32)):
            got = run.run(tokens, want=("logits",))["logits"]
            assert gpu.last_kernel() == "matmul_nt_f32"
            want = graph_oracle.run_graph(pkg, {"tokens": tokens.reshape(1, -1)}, {"seq": tokens.size})["logits"]
            rms = float(np.sqrt((want.astype(np.float64) ** 2).mean()))
            assert got.shape == want.shape and float(np.abs(got - want).max()) <= 1e-5 * rms
    finally:
        run.close()


@pytest.mark.parametrize("wdtype", [be.Q4_0, be.Q8_0])
def test_fused_schedule_counts_steps_and_matches_the_node_by_node_one(gpu, wdtype):
    cfg = DecoderConfig(wdtype=wdtype, **SMALL)
    weights = SyntheticWeights(cfg, 7)
    pkg = aion_file.parse(package_bytes(cfg, weights))
    fused, plain = PackageRunner(gpu, pkg, capacity=cfg.max_seq), PackageRunner(gpu, pkg, capacity=cfg.max_seq, fuse=False)
    try:
        L = cfg.layers
        # node by node: per layer 2 norms, 7 matmuls, 2 ropes, 2 appends (each with its cast), attention, gate, 2 adds
        assert plain.step_count(1) == 1 + 17 * L + 3 and plain.step_count(5) == 1 + 17 * L + 3
        # one new token: qkv+rope+append, attention, o (+residual), norm+gate/up+gelu+down (+residual) per layer
        assert fused.step_count(1) == 1 + 4 * L + 2
        # several tokens: norm+qkv, 2 ropes, 2 appends, attention, o (+residual), norm+gate/up, gate+down (+residual)
        assert fused.step_count(5) == 1 + 9 * L + 2
        prompt = np.random.default_rng(3).integers(0, cfg.vocab, 5).astype(np.int32)
        a, b = fused.run(prompt, want=("next_token", "logits")), plain.run(prompt, want=("next_token", "logits"))
        rms = float(np.sqrt((b["logits"].astype(np.float64) ** 2).mean()))
        # same int8 codes and block dots; an f32 rounding difference can flip a code now and then (see test_gpu_decoder.py)
        assert float(np.abs(a["logits"] - b["logits"]).max()) < 0.1 * rms
        ta, tb = int(a["next_token"][0, -1]), int(b["next_token"][0, -1])
        for _ in range(4):
            a, b = fused.run([ta], want=("next_token", "logits")), plain.run([ta], want=("next_token", "logits"))
            assert float(np.abs(a["logits"] - b["logits"]).max()) < 0.1 * rms
            ta = int(a["next_token"][0, -1])
    finally:
        fused.close(); plain.close()


def test_recorded_decode_program_equals_the_eager_runs(gpu):
    cfg = DecoderConfig(wdtype=be.Q4_0, **SMALL)
    weights = SyntheticWeights(cfg, 11)
    pkg = aion_file.parse(package_bytes(cfg, weights))
    a, b = PackageRunner(gpu, pkg, capacity=cfg.max_seq), PackageRunner(gpu, pkg, capacity=cfg.max_seq)
    try:
        prompt = np.random.default_rng(4).integers(0, cfg.vocab, 9).astype(np.int32)
        ta = int(a.run(prompt)["next_token"][0, -1])
        tb = int(b.run(prompt)["next_token"][0, -1])
        assert ta == tb
        a.begin_decode(ta)
        assert gpu.program_node_count(a.program) > 10
        for step in range(8):
            fed = ta
            ta = a.decode_step()                                           # replayed graph, loop state on the device
            tb = int(b.run([fed])["next_token"][0, -1])                    # the same plan issued eagerly
            gpu.sync()
            assert ta == tb, step
        assert a.pos == b.pos == prompt.size + 8
    finally:
        a.close(); b.close()


def test_sliding_window_package_on_rolling_caches_equals_full_caches(gpu):
    """A sliding-window decoder whose caches are rolling rings of 64 rows must produce what the same model produces
    with caches that hold the whole history: the window (24 back) never reaches past what the ring retains. Bit for
    bit: the same kernels visit the same keys in the same order, only the rows they are read from differ. (A ring
    shorter than the 64-key tile of the MFMA kernels runs on the generic kernel, which does not round q to f16.)"""
    cfg = DecoderConfig(wdtype=be.Q4_0, **SMALL)
    weights = SyntheticWeights(cfg, 13)
    d = dict(layers=cfg.layers, hidden=cfg.hidden, heads=cfg.heads, kv_heads=cfg.kv_heads, head_dim=cfg.head_dim, ffn=cfg.ffn,
             vocab=cfg.vocab, eps=cfg.eps, rope_base=cfg.rope_base, wdtype="q4_0")
    window = (24, 0, 0)
    ring_pkg = aion_file.parse(aion_writer.build_decoder_package(d, weights.blocks, weights.embed(), window=window, retained=24))
    full_pkg = aion_file.parse(aion_writer.build_decoder_package(d, weights.blocks, weights.embed(), window=window))
    assert ring_pkg.role_of_input(4).retained_history_tokens == 24 and full_pkg.role_of_input(4).retained_history_tokens == 0
    # both sides issue the same steps, fused ones included (the one-token q/k/v step appends into rings too)
    ring, full = PackageRunner(gpu, ring_pkg, capacity=64), PackageRunner(gpu, full_pkg, capacity=128)
    assert ring.step_count(1) == full.step_count(1) == 1 + 4 * cfg.layers + 2
    try:
        prompt = np.random.default_rng(2).integers(0, cfg.vocab, 7).astype(np.int32)
        a, b = ring.run(prompt, want=("next_token", "logits")), full.run(prompt, want=("next_token", "logits"))
        assert np.array_equal(a["logits"], b["logits"])
        tok = int(b["next_token"][0, -1])
        for step in range(100):                                  # runs well past the ring's 64 rows
            a, b = ring.run([tok], want=("next_token", "logits")), full.run([tok], want=("next_token", "logits"))
            assert np.array_equal(a["logits"], b["logits"]), step
            tok = int(b["next_token"][0, -1])
        assert ring.pos == 107
    finally:
        ring.close(); full.close()


def test_growing_caches_match_preallocated_ones(gpu):
    """A session whose caches start at 8 rows and grow on the device (8 -> 32 -> 128) must produce the tokens of one
    whose caches were allocated at 128 rows from the start (api/test_sequence_cache.zig:228 "a growable cache matches
    a preallocated one"): growth keeps every row where it was. Logits are compared to f32 rounding, not bit for bit:
    the attention kernels split their key range by the cache's capacity."""
    cfg = DecoderConfig(wdtype=be.Q4_0, **SMALL)
    weights = SyntheticWeights(cfg, 17)
    d = dict(layers=cfg.layers, hidden=cfg.hidden, heads=cfg.heads, kv_heads=cfg.kv_heads, head_dim=cfg.head_dim, ffn=cfg.ffn,
             vocab=cfg.vocab, eps=cfg.eps, rope_base=cfg.rope_base, wdtype="q4_0")
    pkg = aion_file.parse(aion_writer.build_decoder_package(d, weights.blocks, weights.embed(), growable=True))
    fixed_pkg = aion_file.parse(aion_writer.build_decoder_package(d, weights.blocks, weights.embed()))
    assert pkg.role_of_input(4).flags == 3 and fixed_pkg.role_of_input(4).flags == 1
    with pytest.raises(Unsupported):
        PackageRunner(gpu, fixed_pkg, capacity=8, growth=dict(numerator=2, denominator=1))
    grow = PackageRunner(gpu, pkg, capacity=8, growth=dict(numerator=2, denominator=1, max_capacity=128))
    full = PackageRunner(gpu, pkg, capacity=128)
    try:
        prompt = np.random.default_rng(3).integers(0, cfg.vocab, 11).astype(np.int32)      # 11 rows: the first growth, 8 -> 32
        a, b = grow.run(prompt, want=("next_token", "logits")), full.run(prompt, want=("next_token", "logits"))
        assert grow.capacity == 32
        assert np.allclose(a["logits"], b["logits"], atol=2e-4, rtol=1e-4)
        assert np.array_equal(a["next_token"], b["next_token"])
        tok = int(b["next_token"][0, -1])
        # eager single tokens up to the edge of 32, then the recorded program across the second growth
        for step in range(15):
            a, b = grow.run([tok], want=("next_token", "logits")), full.run([tok], want=("next_token", "logits"))
            assert np.allclose(a["logits"], b["logits"], atol=2e-4, rtol=1e-4), step
            assert np.array_equal(a["next_token"], b["next_token"]), step
            tok = int(b["next_token"][0, -1])
        grow.begin_decode(tok); full.begin_decode(tok)
        for step in range(60):
            ta, tb = grow.decode_step(), full.decode_step()
            assert ta == tb, step
        assert grow.capacity == 128 and grow.pos == full.pos == 86
        # the grown caches hold what the preallocated ones hold
        for idx in grow.caches:
            got = gpu.download(grow.caches[idx], np.float16, (128, cfg.kv_heads * cfg.head_dim))
            want = gpu.download(full.caches[idx], np.float16, (128, cfg.kv_heads * cfg.head_dim))
            assert np.allclose(got[:86].astype(np.float32), want[:86].astype(np.float32), atol=4e-3) and not got[86:].any()
        with pytest.raises(ValueError):
            grow.run(np.zeros(60, np.int32))                                            # 146 rows: past the ceiling
    finally:
        grow.close(); full.close()


def test_decode_run_logs_tokens_on_the_device_across_cache_growth(gpu):
    """decode_run: replays back to back with the produced tokens logged on the device (a counter of their own beside the
    loop state) against the same generation one read-back per step; the run crosses a growth of the caches (32 -> 128)
    and a second run goes on where the first stopped."""
    cfg = DecoderConfig(wdtype=be.Q4_0, **SMALL)
    weights = SyntheticWeights(cfg, 23)
    d = dict(layers=cfg.layers, hidden=cfg.hidden, heads=cfg.heads, kv_heads=cfg.kv_heads, head_dim=cfg.head_dim, ffn=cfg.ffn,
             vocab=cfg.vocab, eps=cfg.eps, rope_base=cfg.rope_base, wdtype="q4_0")
    pkg = aion_file.parse(aion_writer.build_decoder_package(d, weights.blocks, weights.embed(), growable=True))
    logged = PackageRunner(gpu, pkg, capacity=32, growth=dict(numerator=2, denominator=1, max_capacity=128))
    stepped = PackageRunner(gpu, pkg, capacity=128)
    try:
        prompt = np.random.default_rng(6).integers(0, cfg.vocab, 9).astype(np.int32)
        a, b = logged.run(prompt, want=("next_token",)), stepped.run(prompt, want=("next_token",))
        tok = int(b["next_token"][0, -1])
        assert int(a["next_token"][0, -1]) == tok
        logged.begin_decode(tok); stepped.begin_decode(tok)
        want = [stepped.decode_step() for _ in range(70)]
        got = logged.decode_run(40) + logged.decode_run(30)
        assert logged.capacity == 128 and logged.pos == stepped.pos == 79
        assert got == want
        assert logged.decode_step() == stepped.decode_step()       # a single step after the runs: the loop state is where it should be
    finally:
        logged.close(); stepped.close()


def test_rolling_caches_grow_for_a_long_run(gpu):
    """A ring of 64 rows (12 retained) asked to take a 60-token run needs 12 + 60 rows: it grows to 256 with its
    retained rows re-placed (storage/manager/grow.zig:107-150), and the session goes on as one that had 256 rows all
    along, also after the positions wrap around the ring. (Both rings are at least one 64-key tile long, so both
    sessions run on the same kernel family from the first run on.)"""
    cfg = DecoderConfig(wdtype=be.Q4_0, **SMALL)
    weights = SyntheticWeights(cfg, 19)
    d = dict(layers=cfg.layers, hidden=cfg.hidden, heads=cfg.heads, kv_heads=cfg.kv_heads, head_dim=cfg.head_dim, ffn=cfg.ffn,
             vocab=cfg.vocab, eps=cfg.eps, rope_base=cfg.rope_base, wdtype="q4_0")
    pkg = aion_file.parse(aion_writer.build_decoder_package(d, weights.blocks, weights.embed(), window=(12, 0, 0), retained=12))
    grow = PackageRunner(gpu, pkg, capacity=64, growth=dict(numerator=2, denominator=1), fuse=False)
    full = PackageRunner(gpu, pkg, capacity=256, fuse=False)
    fixed = PackageRunner(gpu, pkg, capacity=64, fuse=False)
    try:
        rng = np.random.default_rng(4)
        first, second = rng.integers(0, cfg.vocab, 14).astype(np.int32), rng.integers(0, cfg.vocab, 60).astype(np.int32)
        for r in (grow, full, fixed):
            r.run(first)
        with pytest.raises(ValueError):
            fixed.run(second)
        a, b = grow.run(second, want=("next_token", "logits")), full.run(second, want=("next_token", "logits"))
        assert grow.capacity == 256
        assert np.allclose(a["logits"], b["logits"], atol=2e-4, rtol=1e-4)
        tok = int(b["next_token"][0, -1])
        for step in range(200):                                    # positions 74 .. 273: around the ring
            a, b = grow.run([tok], want=("next_token", "logits")), full.run([tok], want=("next_token", "logits"))
            assert np.allclose(a["logits"], b["logits"], atol=2e-4, rtol=1e-4), step
            tok = int(b["next_token"][0, -1])
    finally:
        grow.close(); full.close(); fixed.close()


def test_bench_model_shaped_package_against_the_graph_oracle(gpu, orc):
    """A package in the shape of aion's own bench model (tied row-quantized embedding table gathered from and
    contracted against, scaled embedding, per-head q/k/v norms, norms on the block outputs, local layers with
    sliding windows over rolling caches of constant size beside global layers, soft-capped logits: oracle/aion_writer.py
    build_sandwich_decoder_package) through the package runner, against the node-by-node CPU interpreter
    (oracle/graph_oracle.py) fed the same package. The tolerance is the decoder tests': the GPU may be no further from
    the interpreter than the interpreter is from itself when one operand rounding changes (queries rounded to f16, as
    the MFMA kernels do) - a flipped int8 activation code is worth ~5e-3 of a matmul's output, whatever flipped it;
    and the tokens the interpreter picks wherever its top two logits are further apart than the error."""
    from oracle import graph_oracle
    cfg = dict(layers=3, hidden=256, heads=4, kv_heads=1, head_dim=64, ffn=512, vocab=1024, eps=1e-6, rope_base_local=10000.0,
               rope_base_global=1000000.0, local_window=64, global_every=3, logit_softcap=30.0, wdtype="q4_0")
    E, H, Hkv, D, F, V, W = cfg["hidden"], cfg["heads"], cfg["kv_heads"], cfg["head_dim"], cfg["ffn"], cfg["vocab"], cfg["local_window"]
    rng = np.random.default_rng(23)
    shapes = {"wq": (E, H * D), "wk": (E, Hkv * D), "wv": (E, Hkv * D), "wo": (H * D, E), "wgate": (E, F), "wup": (E, F), "wdown": (F, E)}
    blocks = {"l%d.%s" % (l, n): orc.quantize(orc.Q4_0, (rng.standard_normal(s) * 0.06).astype(np.float32), 0)
              for l in range(cfg["layers"]) for n, s in shapes.items()}
    table = orc.quantize(orc.Q8_0, (rng.standard_normal((V, E)) * 0.05).astype(np.float32), 1)
    gammas = {}
    for l in range(cfg["layers"]):
        for n, width in (("norm_in", E), ("q_norm", D), ("k_norm", D), ("v_norm", D), ("norm_attn", E), ("norm_ffn_in", E), ("norm_ffn", E)):
            # attention runs with scale 1 on normalized heads: gammas of 0.35 on q and k put the scores where a trained
            # model's are (unit gammas give |q.k| up to the head size and a softmax that magnifies every rounding)
            g0 = 0.35 if n in ("q_norm", "k_norm") else 1.0
            gammas["l%d.%s" % (l, n)] = (g0 * (1 + 0.1 * rng.standard_normal(width))).astype(np.float32)
    gammas["norm_f"] = (1 + 0.1 * rng.standard_normal(E)).astype(np.float32)
    pkg = aion_file.parse(aion_writer.build_sandwich_decoder_package(cfg, lambda name: blocks[name], table, gammas))
    T = 128
    run = PackageRunner(gpu, pkg, capacity=T)
    plain = PackageRunner(gpu, pkg, capacity=T, fuse=False)
    caches, rings = {}, []
    for idx, (name, vid) in enumerate(pkg.inputs):
        role = pkg.role_of_input(idx)
        if role.kind == "sequence_cache":
            caches[name] = np.zeros(pkg.shape_of(vid, {"ctx": T, "seq": 1}), np.float16)
            if role.retained_history_tokens:
                rings.append(name)
    assert len(rings) == 4 and len(caches) == 6
    try:
        pos, tok, errs, selfs = 0, None, [], []
        prompt = rng.integers(0, V, 40).astype(np.int32)
        for step in range(1 + 45):                        # 40 prompt tokens, then single tokens past the rings' 64 rows
            tokens = prompt if step == 0 else np.array([tok], np.int32)
            s = tokens.size
            feeds = dict(caches)
            by_role = {"tokens": tokens.reshape(1, s), "positions": np.arange(pos, pos + s, dtype=np.int32).reshape(1, s),
                       "cache_write_index": np.array([pos], np.int32), "cache_visible_end": np.array([pos + s], np.int32)}
            for idx, (name, _vid) in enumerate(pkg.inputs):
                if pkg.role_of_input(idx).kind in by_role:
                    feeds[name] = by_role[pkg.role_of_input(idx).kind]
            want = graph_oracle.run_graph(pkg, feeds, {"seq": s, "ctx": T}, rolling_inputs=rings)
            alt = graph_oracle.run_graph(pkg, feeds, {"seq": s, "ctx": T}, rolling_inputs=rings, round_q_f16=True)
            for name in caches:
                caches[name] = want[name]
            got = run.run(tokens, want=("next_token", "logits"))
            got_plain = plain.run(tokens, want=("next_token", "logits"))
            if step in (0, 1, 30):
                # node by node: every step of the unfused plan against the interpreter ON THE DEVICE'S OWN INPUTS
                # (no amplification between nodes). Prompt, first single token, and a token after the rings wrapped.
                np_t = {"f32": np.float32, "i32": np.int32, "f16": np.float16}
                dev = {vid: gpu.download(buf, np_t[dt], shape) for vid, (buf, shape, dt) in plain.plans[s].values.items()}
                report = graph_oracle.check_nodes(pkg, feeds, {"seq": s, "ctx": T}, dev, rolling_inputs=rings)
                assert len(report) > 50
                for i, op, e in report:
                    assert e < (4e-3 if op == "Attention" else 2e-5), (step, i, op, e)
            ol, gl = want["logits"][0, -1], got["logits"][0, -1]
            rms = float(np.sqrt((ol.astype(np.float64) ** 2).mean()))
            err = float(np.abs(gl - ol).max()) / rms
            errs.append(err)
            selfs.append(float(np.abs(alt["logits"][0, -1] - ol).max()) / rms)
            # the fused schedule against the node-by-node one on the same device: f32 summation order only
            assert float(np.abs(got_plain["logits"][0, -1] - gl).max()) / rms < 2e-3
            top2 = np.sort(ol)[-2:]
            otok = int(want["next_token"][0, -1])
            if float(top2[1] - top2[0]) / rms > 2 * err:
                assert int(got["next_token"][0, -1]) == otok, step
            tok = otok
            pos += s
        say("bench-shaped package: max err/rms %.2e, mean %.2e (interpreter against itself: %.2e, %.2e) over %d runs; steps per token %d (node by node %d)"
            % (max(errs), float(np.mean(errs)), max(selfs), float(np.mean(selfs)), len(errs), run.step_count(1), plain.step_count(1)))
        assert np.mean(errs) < 2 * np.mean(selfs) + 1e-3 and max(errs) < 3 * max(selfs) + 1e-3
        assert np.abs(got["logits"]).max() <= 30.0
        # the head norms, the rotations and the appends of a block are one step, for the prompt and for single tokens
        for s_len in (40, 1):
            names = [fn.__name__ for fn, _a, _k in run.plans[s_len].steps]
            assert names.count("step_headnorm_rope_append") == cfg["layers"]
            assert not any(x in names for x in ("step_rope", "step_append_f16", "step_cast_f32_f16"))
            assert "step_headnorm_rope_append" not in [fn.__name__ for fn, _a, _k in plain.plans[s_len].steps]
        # seven steps per block for a single token (norm + q/k/v, head norms + RoPE + append, attention, o, norm + residual,
        # norm + GeGLU + down, norm + residual) and seven around the blocks
        assert run.step_count(1) <= 7 * cfg["layers"] + 7
        residual_norms = [k for fn, _a, k in run.plans[1].steps if fn.__name__ == "step_rmsnorm" and k.get("residual") is not None]
        assert len(residual_norms) == 2 * cfg["layers"]
        with pytest.raises(ValueError):
            run.run(np.zeros(30, np.int32))               # 63 retained + 30 new rows do not fit a 64-row ring
    finally:
        run.close(); plain.close()
