"""The native step-list executor (Session.execute, backend/backend.zig:42-44) against the same steps issued one by one
through the per-step entry points, whose parity with the CPU oracle the other GPU tests hold: a list must give those
results to the bit, with and without the step patterns it may fold."""
import numpy as np
import pytest

from aion_amd import backend as be
from aion_amd import hip
from aion_amd import session as ss

pytestmark = pytest.mark.gpu

E, HQ, HKV, D, F, V, T = 256, 4, 2, 64, 512, 1000, 32
EPS = 1e-6
SCALE = 0.125


class Layer:
    """Device state of a one-layer decoder program: parameters as aion stores them (packed blocks), a KV cache holding
    `past` tokens and the per-call index tensors. Every run of a comparison starts from a fresh one with the same seed."""

    def __init__(self, gpu, S, past, rolling=False, seed=5, inplace=False):
        """inplace: the two residual adds accumulate into x itself (x = x + o, x = x + dn) instead of writing x1 and x2."""
        rng = np.random.default_rng(seed)
        self.gpu, self.S, self.rolling, self.inplace = gpu, S, rolling, inplace
        self.bufs = {}

        def up(name, a):
            self.bufs[name] = gpu.upload(a)
            return self.bufs[name]

        def weight(name, dtype, k, n, nt=False):
            w = (rng.standard_normal((n, k) if nt else (k, n)) / np.sqrt(k)).astype(np.float32)
            return up(name, be.quantize_blocks(dtype, w, 1 if nt else 0))

        self.table = rng.standard_normal((V, E)).astype(np.float32)
        up("table", self.table)
        for nm in ("g1", "b1", "g2", "b2"):
            up(nm, (1 + 0.1 * rng.standard_normal(E)).astype(np.float32))
        weight("wq", be.Q4_0, E, HQ * D)
        weight("wk", be.Q4_0, E, HKV * D)
        weight("wv", be.Q4_0, E, HKV * D)
        weight("wo", be.Q8_0, HQ * D, E)
        weight("wg", be.Q4_0, E, F)
        weight("wu", be.Q4_0, E, F)
        weight("wd", be.Q4_0, F, E)
        weight("head", be.Q8_0, E, V - V % 8, nt=True)
        self.vocab = V - V % 8
        up("ids", rng.integers(0, V, (1, S)).astype(np.int32))
        up("pos", (past + np.arange(S)).astype(np.int32).reshape(1, S))
        up("widx", np.array([past], np.int32))
        up("len", np.array([past + S], np.int32))
        up("step", np.array([S], np.int32))
        cache = np.zeros((1, T, HKV, D), np.float16)
        cache[:, :min(past, T)] = rng.standard_normal((1, min(past, T), HKV, D)).astype(np.float16)
        up("kc", cache)
        up("vc", np.roll(cache, 1, axis=3))
        for nm, n in (("x", S * E), ("h", S * E), ("q", S * HQ * D), ("k", S * HKV * D), ("v", S * HKV * D), ("qr", S * HQ * D),
                      ("kr", S * HKV * D), ("att", S * HQ * D), ("o", S * E), ("x1", S * E), ("h2", S * E), ("gt", S * F), ("upj", S * F),
                      ("gg", S * F), ("dn", S * E), ("x2", S * E), ("logits", S * self.vocab)):
            self.bufs[nm] = gpu.zeros(n * 4)
        self.bufs["k16"] = gpu.zeros(S * HKV * D * 2)
        self.bufs["v16"] = gpu.zeros(S * HKV * D * 2)
        self.bufs["out_ids"] = gpu.zeros(S * 4)
        if inplace:
            for nm in ("x1", "x2"):
                self.bufs.pop(nm).free()
                self.bufs[nm] = self.bufs["x"].view(0)

    def free(self):
        for b in self.bufs.values():
            b.free()

    # tensors that every form of the program must write (the workspace ones may be folded away)
    KEPT = {"x": np.float32, "q": np.float32, "k": np.float32, "v": np.float32, "qr": np.float32, "kr": np.float32, "kc": np.float16,
            "vc": np.float16, "att": np.float32, "o": np.float32, "x1": np.float32, "gt": np.float32, "upj": np.float32, "dn": np.float32,
            "x2": np.float32, "logits": np.float32, "out_ids": np.int32, "pos": np.int32, "widx": np.int32, "len": np.int32}
    WORKSPACE = {"h": np.float32, "h2": np.float32, "gg": np.float32, "k16": np.float16, "v16": np.float16}

    def results(self, names):
        self.gpu.sync()
        kinds = {**self.KEPT, **self.WORKSPACE}
        return {n: self.bufs[n].numpy(kinds[n]) for n in names}

    # with lean=True these are workspace tensors as well, as in a compiled program, where only the block's outputs survive
    LEAN = ("q", "k", "v", "kr", "gt", "upj", "o", "dn")

    def steps(self, casts_first=False, lean=False):
        """The program as step records."""
        b, S = self.bufs, self.S
        t = lambda nm, dt, shape, **kw: ss.tensor(b[nm], dt, shape, **kw)  # noqa: E731

        def f(nm, *shape, **kw):
            if lean and nm in self.LEAN:
                kw["workspace"] = True
            return t(nm, be.F32, shape, **kw)
        i = lambda nm, *shape: t(nm, be.I32, shape)                        # noqa: E731
        kc = t("kc", be.F16, (1, T, HKV, D), rolling=self.rolling)
        vc = t("vc", be.F16, (1, T, HKV, D), rolling=self.rolling)
        p = ss.Steps()
        p.gather_rows(f("table", V, E), i("ids", 1, S), f("x", 1, S, E))
        p.rmsnorm(f("x", 1, S, E), f("g1", E), f("b1", E), f("h", 1, S, E, workspace=True), EPS)
        p.matmul(f("h", 1, S, E, workspace=True), t("wq", be.Q4_0, (E, HQ * D)), f("q", 1, S, HQ * D))
        p.matmul(f("h", 1, S, E, workspace=True), t("wk", be.Q4_0, (E, HKV * D)), f("k", 1, S, HKV * D))
        p.matmul(f("h", 1, S, E, workspace=True), t("wv", be.Q4_0, (E, HKV * D)), f("v", 1, S, HKV * D))
        p.rope1d(f("q", 1, S, HQ, D), i("pos", 1, S), f("qr", 1, S, HQ, D))
        p.rope1d(f("k", 1, S, HKV, D), i("pos", 1, S), f("kr", 1, S, HKV, D))
        k16 = t("k16", be.F16, (1, S, HKV, D), workspace=True)
        v16 = t("v16", be.F16, (1, S, HKV, D), workspace=True)
        if casts_first:        # both casts ahead of both appends: nothing to fold, same results
            p.cast(f("kr", 1, S, HKV, D), k16)
            p.cast(f("v", 1, S, HKV, D), v16)
            p.sequence_append(kc, k16, i("widx", 1))
            p.sequence_append(vc, v16, i("widx", 1))
        else:
            p.cast(f("kr", 1, S, HKV, D), k16)
            p.sequence_append(kc, k16, i("widx", 1))
            p.cast(f("v", 1, S, HKV, D), v16)
            p.sequence_append(vc, v16, i("widx", 1))
        p.attention(f("qr", 1, S, HQ, D), kc, vc, f("att", 1, S, HQ, D), SCALE, query_positions=i("pos", 1, S), kv_lengths=i("len", 1))
        p.matmul(f("att", 1, S, HQ * D), t("wo", be.Q8_0, (HQ * D, E)), f("o", 1, S, E))
        p.elemwise_binary(ss.ADD, f("x", 1, S, E), f("o", 1, S, E), f("x1", 1, S, E))
        p.rmsnorm(f("x1", 1, S, E), f("g2", E), f("b2", E), f("h2", 1, S, E, workspace=True), EPS)
        p.matmul(f("h2", 1, S, E, workspace=True), t("wg", be.Q4_0, (E, F)), f("gt", 1, S, F))
        p.matmul(f("h2", 1, S, E, workspace=True), t("wu", be.Q4_0, (E, F)), f("upj", 1, S, F))
        p.elemwise_binary(ss.GATE, f("gt", 1, S, F), f("upj", 1, S, F), f("gg", 1, S, F, workspace=True), act=ss.GELU)
        p.matmul(f("gg", 1, S, F, workspace=True), t("wd", be.Q4_0, (F, E)), f("dn", 1, S, E), alpha=0.5)
        p.elemwise_binary(ss.ADD, f("x1", 1, S, E), f("dn", 1, S, E), f("x2", 1, S, E))
        p.matmul_nt(f("x2", 1, S, E), t("head", be.Q8_0, (self.vocab, E)), f("logits", 1, S, self.vocab))
        p.argmax(f("logits", 1, S, self.vocab), i("out_ids", 1, S), axis=2)
        # the decode counters move on the device (i32 adds): positions by scalar broadcast is not i32 territory, so one add each
        p.elemwise_binary(ss.ADD, i("widx", 1), i("step", 1), i("widx", 1))
        p.elemwise_binary(ss.ADD, i("len", 1), i("step", 1), i("len", 1))
        return p

    def run_direct(self):
        """The same steps through the per-step entry points."""
        g, b, S = self.gpu, self.bufs, self.S
        w = {nm: g.weight_from_device(dt, be.KMAJOR_KN, n, k, b[nm]) for nm, dt, k, n in (
            ("wq", be.Q4_0, E, HQ * D), ("wk", be.Q4_0, E, HKV * D), ("wv", be.Q4_0, E, HKV * D), ("wo", be.Q8_0, HQ * D, E),
            ("wg", be.Q4_0, E, F), ("wu", be.Q4_0, E, F), ("wd", be.Q4_0, F, E))}
        w["head"] = g.weight_from_device(be.Q8_0, be.ROWS_NK, self.vocab, E, b["head"])
        g.step_gather_rows(be.F32, b["x"], b["table"], b["ids"], S, E, V)
        g.step_rmsnorm(b["h"], b["x"], b["g1"], S, E, EPS, beta=b["b1"])
        for nm, out in (("wq", "q"), ("wk", "k"), ("wv", "v")):
            g.step_matmul(w[nm], b["h"], S, b[out])
        g.step_rope(b["qr"], b["q"], b["pos"], 1, S, HQ, D)
        g.step_rope(b["kr"], b["k"], b["pos"], 1, S, HKV, D)
        g.step_cast_f32_f16(b["k16"], b["kr"], S * HKV * D)
        g.step_sequence_append(be.F16, b["kc"], b["k16"], b["widx"], 1, S, T, HKV * D, rolling=self.rolling)
        g.step_cast_f32_f16(b["v16"], b["v"], S * HKV * D)
        g.step_sequence_append(be.F16, b["vc"], b["v16"], b["widx"], 1, S, T, HKV * D, rolling=self.rolling)
        g.step_attention(b["att"], b["qr"], b["kc"], b["vc"], (1, S, T, HQ, HKV, D, D), SCALE, query_positions=b["pos"], kv_lengths=b["len"],
                         rolling=self.rolling)
        g.step_matmul(w["wo"], b["att"], S, b["o"])
        g.step_binary("add", b["x1"], b["x"], b["o"], S * E)
        g.step_rmsnorm(b["h2"], b["x1"], b["g2"], S, E, EPS, beta=b["b2"])
        g.step_matmul(w["wg"], b["h2"], S, b["gt"])
        g.step_matmul(w["wu"], b["h2"], S, b["upj"])
        g.step_gate_gelu(b["gg"], b["gt"], b["upj"], S * F)
        g.step_matmul(w["wd"], b["gg"], S, b["dn"], alpha=0.5)
        g.step_binary("add", b["x2"], b["x1"], b["dn"], S * E)
        g.step_matmul(w["head"], b["x2"], S, b["logits"])
        g.step_argmax(b["out_ids"], b["logits"], S, self.vocab)
        g.step_add_i32(b["widx"], b["widx"], b["step"], 1)
        g.step_add_i32(b["len"], b["len"], b["step"], 1)
        g.sync()
        for x in w.values():
            x.free()


def _same(a, b, names):
    for n in names:
        assert np.array_equal(a[n].view(np.uint8), b[n].view(np.uint8)), n


@pytest.mark.parametrize("S,past,rolling", [(1, 9, False), (5, 0, False), (12, 3, False), (3, 40, True)])
def test_a_decoder_layer_as_a_step_list_equals_the_steps_issued_one_by_one(gpu, S, past, rolling):
    """One row (the GEMV routes), up to eight rows, more than eight (the GEMM), and a rolling cache that has wrapped."""
    every = list(Layer.KEPT) + list(Layer.WORKSPACE)
    ref = Layer(gpu, S, past, rolling)
    ref.run_direct()
    want = ref.results(every)
    ref.free()
    assert want["out_ids"].min() >= 0 and np.abs(want["logits"]).max() > 0
    assert want["widx"][0] == past + S and want["len"][0] == past + 2 * S

    sess = ss.Session(gpu)
    # step by step: every tensor, the workspace ones included
    sess.set_fusion(0)
    one = Layer(gpu, S, past, rolling)
    prog = one.steps()
    sess.execute(prog)
    calls_plain = sess.stats()[0]
    assert calls_plain == len(prog.records)
    _same(one.results(every), want, every)
    one.free()
    sess.retire_resources()

    # sibling matmuls in one call: still every tensor, fewer calls
    sess.set_fusion(ss.FUSE_SIBLINGS)
    sib = Layer(gpu, S, past, rolling)
    sess.execute(sib.steps())
    assert sess.stats()[0] == calls_plain - 2 - 1          # q/k/v: three steps in one call; gate/up: two in one
    _same(sib.results(every), want, every)
    sib.free()
    sess.retire_resources()

    # all patterns: the workspace tensors the patterns fold are not written, everything else is the same to the bit
    sess.set_fusion(ss.FUSE_SIBLINGS | ss.FUSE_WORKSPACE)
    fused = Layer(gpu, S, past, rolling)
    sess.execute(fused.steps())
    # rmsnorm + q/k/v -> 1 call (4 steps), cast + append -> 1 call (x2), rmsnorm + gate/up -> 1 call (3 steps), gate + down -> 1 call
    assert sess.stats()[0] == calls_plain - 3 - 1 - 1 - 2 - 1
    got = fused.results(every)
    _same(got, want, Layer.KEPT)
    for n in Layer.WORKSPACE:
        assert not got[n].any(), n                          # folded away: still the zeros the buffers started with
    fused.free()
    sess.retire_resources()                                 # the weights are keyed by tensor address: retired with their tensors

    # every intermediate of the two blocks a workspace tensor: one row runs the attention block's input side as one call
    # (ten steps) and the feed-forward block as one (five steps); more rows run the smaller patterns as before
    lean = Layer(gpu, S, past, rolling)
    for order in (False, True):
        sess.execute(lean.steps(lean=True, casts_first=order))
        # more rows: norm + q/k/v (4 steps, 1 call), the six rope / cast / append steps in either order (1 call), norm + gate / up
        # (3 steps, 1 call), gate + down (2 steps, 1 call)
        # (a rolling cache has no one-call form of the six: there the cast + append pairs fold where they stand side by side)
        tail = 5 if not rolling else (0 if order else 2)
        assert sess.stats()[0] == (calls_plain - 9 - 4 if S == 1 else calls_plain - 3 - tail - 2 - 1)
        got = lean.results(every)
        if S == 1:
            folded = ("q", "k", "v", "kr", "gt", "upj")      # o and dn feed adds that write elsewhere: still written
            _same(got, want, [n for n in Layer.KEPT if n not in folded and n not in ("widx", "len")])
            for n in list(Layer.WORKSPACE) + list(folded):
                assert not got[n].any(), n
        else:
            gone = ["kr", "k16", "v16"] if not rolling else ([] if order else ["k16", "v16"])
            _same(got, want, [n for n in Layer.KEPT if n not in ["widx", "len"] + gone])
            for n in ["h", "h2", "gg"] + gone:
                assert not got[n].any(), n
        # the second pass appends the same rows at the same place: put the counters back
        gpu.write(lean.bufs["widx"], np.array([past], np.int32))
        gpu.write(lean.bufs["len"], np.array([past + S], np.int32))
    lean.free()
    sess.retire_resources()

    # the residual adds accumulate in place (x = x + o, x = x + dn): the matmul in front of each writes x with beta 1
    ref = Layer(gpu, S, past, rolling, inplace=True)
    ref.run_direct()
    want_inplace = ref.results(every)
    ref.free()
    acc = Layer(gpu, S, past, rolling, inplace=True)
    sess.execute(acc.steps(lean=True))
    assert sess.stats()[0] == (calls_plain - 15 if S == 1 else (calls_plain - 13 if not rolling else calls_plain - 10))
    got = acc.results(every)
    folded = ("o", "dn") + (("q", "k", "v", "kr", "gt", "upj") if S == 1 else (("kr",) if not rolling else ()))
    _same(got, want_inplace, [n for n in Layer.KEPT if n not in folded])
    for n in list(Layer.WORKSPACE) + list(folded):
        assert not got[n].any(), n
    acc.free()
    sess.retire_resources()

    # both casts ahead of both appends: the cast pattern does not apply, the f16 rows are written, the results do not move
    other = Layer(gpu, S, past, rolling)
    sess.execute(other.steps(casts_first=True))
    got = other.results(every)
    _same(got, want, list(Layer.KEPT) + ["k16", "v16"])
    other.free()
    sess.close()


def test_a_workspace_tensor_that_is_read_later_is_written(gpu):
    """The norm's output feeds the matmul right behind it and an add further down: it may not be folded away."""
    rng = np.random.default_rng(11)
    S = 1
    x = rng.standard_normal((S, E)).astype(np.float32)
    g = rng.standard_normal(E).astype(np.float32)
    b0 = rng.standard_normal(E).astype(np.float32)
    w = be.quantize_blocks(be.Q4_0, (rng.standard_normal((E, E)) / 16).astype(np.float32), 0)
    xb, gb, bb, wb = gpu.upload(x), gpu.upload(g), gpu.upload(b0), gpu.upload(w)
    h, y, z = gpu.zeros(S * E * 4), gpu.zeros(S * E * 4), gpu.zeros(S * E * 4)
    f = lambda buf, ws=False: ss.tensor(buf, be.F32, (S, E), workspace=ws)  # noqa: E731
    sess = ss.Session(gpu)

    def program(with_later_reader):
        p = ss.Steps()
        p.rmsnorm(f(xb), ss.tensor(gb, be.F32, (E,)), ss.tensor(bb, be.F32, (E,)), f(h, True), EPS)
        p.matmul(f(h, True), ss.tensor(wb, be.Q4_0, (E, E)), f(y))
        if with_later_reader:
            p.elemwise_binary(ss.ADD, f(y), f(h, True), f(z))
        return p

    sess.execute(program(True))
    assert sess.stats()[0] == 3
    hv, yv, zv = h.numpy(np.float32), y.numpy(np.float32), z.numpy(np.float32)
    assert hv.any() and np.array_equal(zv, yv + hv)
    gpu.write(h, np.zeros(S * E, np.float32))
    sess.execute(program(False))
    assert sess.stats()[0] == 1 and not h.numpy(np.float32).any()
    assert np.array_equal(y.numpy(np.float32), yv)
    # the same list with the norm's output not marked as workspace: written
    p = ss.Steps()
    p.rmsnorm(f(xb), ss.tensor(gb, be.F32, (E,)), ss.tensor(bb, be.F32, (E,)), f(h), EPS)
    p.matmul(f(h), ss.tensor(wb, be.Q4_0, (E, E)), f(y))
    sess.execute(p)
    assert sess.stats()[0] == 2 and np.array_equal(h.numpy(np.float32), hv)
    sess.close()
    for buf in (xb, gb, bb, wb, h, y, z):
        buf.free()


def test_a_list_is_checked_as_a_whole_before_anything_runs(gpu):
    rng = np.random.default_rng(12)
    x = rng.standard_normal(64).astype(np.float32)
    xb, out = gpu.upload(x), gpu.upload(np.full(64, 7.0, np.float32))
    f = lambda buf, n=64: ss.tensor(buf, be.F32, (n,))  # noqa: E731
    sess = ss.Session(gpu)
    # Softmax (tag 3) is not a step of this device: Unsupported, and the unary in front of it has not run
    p = ss.Steps()
    p.unary(ss.RELU, f(xb), f(out))
    p.raw(3, f(out), [f(xb)])
    with pytest.raises(be.AionHipError) as e:
        sess.execute(p)
    assert e.value.status == hip.UNSUPPORTED and "step 1" in str(e.value)
    assert np.array_equal(out.numpy(np.float32), np.full(64, 7.0, np.float32))
    # log is the one UnaryOp without a device form; a comparison on i32 and an unknown broadcast likewise
    for bad in (lambda q: q.unary(ss.LOG, f(xb), f(out)),
                lambda q: q.elemwise_binary(4, ss.tensor(xb, be.I32, (64,)), ss.tensor(xb, be.I32, (64,)), ss.tensor(out, be.I32, (64,))),
                lambda q: q.elemwise_binary(ss.ADD, f(xb), f(out), f(out), broadcast=ss.GENERIC),
                lambda q: q.elemwise_binary(ss.GATE, f(xb), f(out), f(out), act=ss.SILU),
                lambda q: q.argmax(ss.tensor(xb, be.F32, (8, 8)), ss.tensor(out, be.I32, (8,)), axis=0),
                lambda q: q.gather(ss.tensor(xb, be.F32, (8, 8)), ss.tensor(out, be.I32, (2,)), f(out, 16), axis=1),
                lambda q: q.cast(f(xb), ss.tensor(out, be.I32, (64,)))):
        q = ss.Steps()
        bad(q)
        with pytest.raises(be.AionHipError) as e:
            sess.execute(q)
        assert e.value.status == hip.UNSUPPORTED
    # shapes that do not agree are invalid arguments, as a program that fails validation (runtime/executable.zig:413-470)
    for bad in (lambda q: q.unary(ss.RELU, f(xb), f(out, 32)),
                lambda q: q.matmul(ss.tensor(xb, be.F32, (1, 64)), ss.tensor(xb, be.Q4_0, (32, 64)), ss.tensor(out, be.F32, (1, 64))),
                lambda q: q.rmsnorm(ss.tensor(xb, be.F32, (2, 32)), f(out, 16), None, ss.tensor(out, be.F32, (2, 32)), EPS),
                lambda q: q.copy(f(xb), f(out, 32)),
                lambda q: q.transfer_to_host(f(xb), np.zeros(8, np.float32)),
                # limits of the entry points behind the tags, found before the first launch as well
                lambda q: q.matmul(ss.tensor(xb, be.F32, (1, 48)), ss.tensor(xb, be.Q4_0, (48, 32)), ss.tensor(out, be.F32, (1, 32))),
                lambda q: q.rmsnorm(ss.tensor(xb, be.F32, (2, 32)), f(out, 32), None, ss.tensor(out, be.F32, (2, 32)), 0.0),
                lambda q: q.rope1d(ss.tensor(xb, be.F32, (1, 1, 4, 3)), ss.tensor(xb, be.I32, (1, 1)), ss.tensor(out, be.F32, (1, 1, 4, 3))),
                lambda q: q.rope1d(ss.tensor(xb, be.F32, (1, 1, 2, 8)), ss.tensor(xb, be.I32, (1, 1)), ss.tensor(out, be.F32, (1, 1, 2, 8)),
                                   rope_proportion=1.5),
                lambda q: q.gather(ss.tensor(xb, be.Q8_0, (4, 16)), ss.tensor(xb, be.I32, (2,)), f(out, 32)),
                lambda q: q.attention(ss.tensor(xb, be.F32, (1, 1, 3, 8)), ss.tensor(xb, be.F16, (1, 2, 2, 8)), ss.tensor(xb, be.F16, (1, 2, 2, 8)),
                                      ss.tensor(out, be.F32, (1, 1, 3, 8)), 0.1)):
        q = ss.Steps()
        q.unary(ss.RELU, f(xb), f(out))          # a valid step in front: it may not have run when the list is refused
        bad(q)
        with pytest.raises(be.AionHipError) as e:
            sess.execute(q)
        assert e.value.status == hip.INVALID_ARGUMENT and "step 1" in str(e.value)
        assert np.array_equal(out.numpy(np.float32), np.full(64, 7.0, np.float32))
    sess.execute(ss.Steps())          # an empty list is a program with nothing to do
    with pytest.raises(be.AionHipError) as e:
        sess.set_fusion(8)
    assert e.value.status == hip.INVALID_ARGUMENT
    sess.close()
    xb.free()
    out.free()


def test_transfers_copy_and_elementwise_steps(gpu, orc):
    """Transfer in, the broadcast forms of ElemwiseBinary, Unary, Copy, Gather over a q8_0 table, Transfer out."""
    rng = np.random.default_rng(13)
    a = rng.standard_normal((3, 5, 64)).astype(np.float32)
    suffix = (rng.standard_normal((5, 64)) + 3).astype(np.float32)
    scalar = np.array([1.75], np.float32)
    table = rng.standard_normal((40, 64)).astype(np.float32)
    ids = rng.integers(0, 40, (15,)).astype(np.int32)
    ab, sb, cb, tb, ib = gpu.zeros(a.nbytes), gpu.upload(suffix), gpu.upload(scalar), gpu.upload(be.quantize_blocks(be.Q8_0, table, 1)), gpu.upload(ids)
    t1, t2, t3, t4 = (gpu.zeros(a.nbytes) for _ in range(4))
    f = lambda buf: ss.tensor(buf, be.F32, (3, 5, 64))  # noqa: E731
    got_div, got_sig, got_rows = np.zeros_like(a), np.zeros_like(a), np.zeros((15, 64), np.float32)
    p = ss.Steps()
    p.transfer_to_device(a, f(ab))
    p.elemwise_binary(ss.DIV, f(ab), ss.tensor(sb, be.F32, (5, 64)), f(t1), broadcast=ss.SUFFIX_B)
    p.elemwise_binary(ss.SUB, f(t1), ss.tensor(cb, be.F32, (1,)), f(t2), broadcast=ss.SCALAR_B)
    p.unary(ss.SIGMOID, f(t2), f(t3))
    p.copy(f(t3), f(t4))
    p.gather(ss.tensor(tb, be.Q8_0, (40, 64)), ss.tensor(ib, be.I32, (15,)), ss.tensor(t1, be.F32, (15, 64)))
    p.transfer_to_host(f(t2), got_div)
    p.transfer_to_host(f(t4), got_sig)
    p.transfer_to_host(ss.tensor(t1, be.F32, (15, 64)), got_rows)
    sess = ss.Session(gpu)
    sess.execute(p)
    assert np.array_equal(got_div, orc.binary("sub", orc.binary("div", a, suffix), scalar))
    assert np.allclose(got_sig, orc.unary("sigmoid", got_div), rtol=0, atol=2e-6)
    assert np.array_equal(got_rows, orc.dequantize(be.Q8_0, orc.quantize(be.Q8_0, table, 1), table.shape, 1)[ids])
    sess.close()
    for buf in (ab, sb, cb, tb, ib, t1, t2, t3, t4):
        buf.free()


def test_retire_drops_the_relaid_weights_and_a_list_records_as_a_program(gpu):
    S, past = 1, 6
    sess = ss.Session(gpu)
    L = Layer(gpu, S, past)
    prog = L.steps()
    sess.execute(prog)
    first = L.results(["logits", "out_ids", "kc"])
    _, n_w, w_bytes = sess.stats()
    assert n_w == 8 and w_bytes > 0
    # the same list again: no weight is built twice
    sess.execute(prog)
    assert sess.stats()[1] == 8
    sess.retire_resources()
    assert sess.stats()[1:] == (0, 0)
    L.free()

    # recorded: once eagerly (weights, scratch), then the list between program_begin and program_end, replayed per token
    L = Layer(gpu, S, past)
    sess.execute(L.steps())
    want1 = L.results(["logits", "out_ids"])
    _same(want1, first, ["logits", "out_ids"])
    gpu.write(L.bufs["ids"], want1["out_ids"].reshape(1, S))
    gpu.write(L.bufs["pos"], np.array([[past + 1]], np.int32))
    program = gpu.record_program(lambda: sess.execute(L.steps()))
    assert gpu.program_node_count(program) >= sess.stats()[0]          # a call is one launch or a few
    replayed = []
    for t in range(3):
        gpu.program_execute(program)
        r = L.results(["logits", "out_ids", "widx", "len"])
        assert r["widx"][0] == past + 2 + t and r["len"][0] == past + 3 + t
        replayed.append(r)
        gpu.write(L.bufs["ids"], r["out_ids"].reshape(1, S))
        gpu.write(L.bufs["pos"], np.array([[past + 2 + t]], np.int32))
    gpu.program_destroy(program)
    L.free()
    sess.retire_resources()

    # the same three tokens eagerly
    L = Layer(gpu, S, past)
    sess.execute(L.steps())
    r = L.results(["out_ids"])
    for t in range(3):
        gpu.write(L.bufs["ids"], r["out_ids"].reshape(1, S))
        gpu.write(L.bufs["pos"], np.array([[past + 1 + t]], np.int32))
        sess.execute(L.steps())
        r = L.results(["logits", "out_ids"])
        _same(r, replayed[t], ["logits", "out_ids"])
    L.free()
    # a weight whose first use would fall inside a recording is refused, and the recording is dropped
    sess.retire_resources()
    L = Layer(gpu, S, past)
    with pytest.raises(be.AionHipError) as e:
        gpu.record_program(lambda: sess.execute(L.steps()))
    assert e.value.status == hip.INVALID_ARGUMENT and "eagerly" in str(e.value)
    sess.execute(L.steps())          # the context executes eagerly again
    _same(L.results(["logits"]), first, ["logits"])
    L.free()
    sess.close()


def test_a_fold_is_skipped_when_an_output_lies_over_an_input_it_would_still_read(gpu):
    """h = RMSNorm(x); x = h @ Wq (over x itself); k = h @ Wk. Step by step the norm is finished before x is overwritten; folded
    into one launch the norm would be recomputed from an x that other workgroups are already overwriting. The executor must
    see the overlap and keep the norm a step of its own (the two matmuls may still share a launch: they read h)."""
    rng = np.random.default_rng(21)
    x = rng.standard_normal((1, E)).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(E)).astype(np.float32)
    wq = be.quantize_blocks(be.Q4_0, (rng.standard_normal((E, E)) / 16).astype(np.float32), 0)
    wk = be.quantize_blocks(be.Q4_0, (rng.standard_normal((E, E)) / 16).astype(np.float32), 0)
    gb, wqb, wkb = gpu.upload(g), gpu.upload(wq), gpu.upload(wk)
    got = {}
    sess = ss.Session(gpu)
    for fusion in (0, ss.FUSE_SIBLINGS | ss.FUSE_WORKSPACE):
        xb, h, k = gpu.upload(x), gpu.zeros(E * 4), gpu.zeros(E * 4)
        f = lambda buf, ws=False: ss.tensor(buf, be.F32, (1, E), workspace=ws)  # noqa: E731
        p = ss.Steps()
        p.rmsnorm(f(xb), ss.tensor(gb, be.F32, (E,)), None, f(h, True), EPS)
        p.matmul(f(h, True), ss.tensor(wqb, be.Q4_0, (E, E)), f(xb))
        p.matmul(f(h, True), ss.tensor(wkb, be.Q4_0, (E, E)), f(k))
        sess.set_fusion(fusion)
        sess.execute(p)
        assert sess.stats()[0] == (3 if fusion == 0 else 2)
        got[fusion] = (xb.numpy(np.float32), k.numpy(np.float32), h.numpy(np.float32))
        for buf in (xb, h, k):
            buf.free()
    for a, b in zip(got[0], got[3]):
        assert np.array_equal(a, b)
    assert got[0][2].any()                     # the norm's output was written both times
    # the same with the gate: act(a) * b -> matmul written over a
    a0, b0 = rng.standard_normal((1, E)).astype(np.float32), rng.standard_normal((1, E)).astype(np.float32)
    got = {}
    for fusion in (0, ss.FUSE_SIBLINGS | ss.FUSE_WORKSPACE):
        ab, bb, t = gpu.upload(a0), gpu.upload(b0), gpu.zeros(E * 4)
        p = ss.Steps()
        p.elemwise_binary(ss.GATE, f(ab), f(bb), f(t, True), act=ss.GELU)
        p.matmul(f(t, True), ss.tensor(wqb, be.Q4_0, (E, E)), f(ab))
        sess.set_fusion(fusion)
        sess.execute(p)
        assert sess.stats()[0] == 2
        got[fusion] = ab.numpy(np.float32)
        for buf in (ab, bb, t):
            buf.free()
    assert np.array_equal(got[0], got[3])
    sess.close()
    for buf in (gb, wqb, wkb):
        buf.free()


@pytest.mark.parametrize("B,S,rolling,with_beta,order", [(1, 1, False, True, 0), (2, 3, False, False, 1), (1, 5, True, True, 2)])
def test_head_norms_rope_and_appends_fold_into_one_call(gpu, B, S, rolling, with_beta, order):
    """The cache side of a block whose heads are normalized (src/bench/models.zig:455-473): nine steps, one call, the
    bits of the nine; the three chains in different step orders."""
    Hq, Hkv, Dh, Tc = 4, 2, 64, 8
    rng = np.random.default_rng(31 + order)
    q = rng.standard_normal((B, S, Hq, Dh)).astype(np.float32)
    k = rng.standard_normal((B, S, Hkv, Dh)).astype(np.float32)
    v = rng.standard_normal((B, S, Hkv, Dh)).astype(np.float32)
    start = 6 if rolling else 2
    pos = np.tile(np.arange(start, start + S, dtype=np.int32), (B, 1))
    seed = rng.standard_normal((B, Tc, Hkv, Dh)).astype(np.float16)
    const = {nm: gpu.upload(a) for nm, a in (("q", q), ("k", k), ("v", v), ("pos", pos), ("widx", np.full(B, start, np.int32)))}
    for nm in ("gq", "gk", "gv"):
        const[nm] = gpu.upload((1 + 0.2 * rng.standard_normal(Dh)).astype(np.float32))
    for nm in ("bq", "bk", "bv"):
        const[nm] = gpu.upload((0.1 * rng.standard_normal(Dh)).astype(np.float32)) if with_beta else None
    sess = ss.Session(gpu)
    got = {}
    for fusion in (0, ss.FUSE_SIBLINGS | ss.FUSE_WORKSPACE):
        w = {nm: gpu.zeros(4 * B * S * h * Dh) for nm, h in (("nq", Hq), ("nk", Hkv), ("nv", Hkv), ("qr", Hq), ("kr", Hkv))}
        w["k16"], w["v16"] = gpu.zeros(2 * B * S * Hkv * Dh), gpu.zeros(2 * B * S * Hkv * Dh)
        w["kc"], w["vc"] = gpu.upload(seed), gpu.upload(seed[:, ::-1].copy())
        f = lambda buf, h, ws=False: ss.tensor(buf, be.F32, (B, S, h, Dh), workspace=ws)  # noqa: E731
        vec = lambda nm: ss.tensor(const[nm], be.F32, (Dh,)) if const[nm] is not None else None  # noqa: E731
        k16 = ss.tensor(w["k16"], be.F16, (B, S, Hkv, Dh), workspace=True)
        v16 = ss.tensor(w["v16"], be.F16, (B, S, Hkv, Dh), workspace=True)
        kc = ss.tensor(w["kc"], be.F16, (B, Tc, Hkv, Dh), rolling=rolling)
        vc = ss.tensor(w["vc"], be.F16, (B, Tc, Hkv, Dh), rolling=rolling)
        posr, widx = ss.tensor(const["pos"], be.I32, (B, S)), ss.tensor(const["widx"], be.I32, (B,))
        parts = {
            "nq": lambda p: p.rmsnorm(f(const["q"], Hq), vec("gq"), vec("bq"), f(w["nq"], Hq, True), EPS),
            "nk": lambda p: p.rmsnorm(f(const["k"], Hkv), vec("gk"), vec("bk"), f(w["nk"], Hkv, True), EPS),
            "nv": lambda p: p.rmsnorm(f(const["v"], Hkv), vec("gv"), vec("bv"), f(w["nv"], Hkv, True), EPS),
            "rq": lambda p: p.rope1d(f(w["nq"], Hq, True), posr, f(w["qr"], Hq), rope_proportion=0.5),
            "rk": lambda p: p.rope1d(f(w["nk"], Hkv, True), posr, f(w["kr"], Hkv, True), rope_proportion=0.5),
            "ck": lambda p: p.cast(f(w["kr"], Hkv, True), k16),
            "cv": lambda p: p.cast(f(w["nv"], Hkv, True), v16),
            "ak": lambda p: p.sequence_append(kc, k16, widx),
            "av": lambda p: p.sequence_append(vc, v16, widx),
        }
        orders = (("nq", "nk", "nv", "rq", "rk", "ck", "ak", "cv", "av"), ("nk", "rk", "ck", "ak", "nv", "cv", "av", "nq", "rq"),
                  ("nv", "nq", "rq", "cv", "nk", "av", "rk", "ck", "ak"))
        p = ss.Steps()
        for nm in orders[order]:
            parts[nm](p)
        # a reader of the rotated queries behind the pattern, as the attention step would be
        p.unary(ss.RELU, f(w["qr"], Hq), f(w["nq"], Hq, True))
        sess.set_fusion(fusion)
        sess.execute(p)
        assert sess.stats()[0] == (10 if fusion == 0 else 2)
        got[fusion] = {nm: w[nm].numpy(np.float16 if nm in ("kc", "vc", "k16", "v16") else np.float32) for nm in w}
        for buf in w.values():
            buf.free()
    for nm in ("qr", "kc", "vc", "nq"):
        assert np.array_equal(got[0][nm].view(np.uint8), got[3][nm].view(np.uint8)), nm
    assert got[0]["k16"].any() and not got[3]["k16"].any() and not got[3]["kr"].any() and not got[3]["nv"].any()
    rows = [(start + s) % Tc if rolling else start + s for s in range(S)]
    kc_got = got[3]["kc"].reshape(B, Tc, Hkv, Dh)
    untouched = [t for t in range(Tc) if t not in rows]
    assert np.array_equal(kc_got[:, untouched], seed[:, untouched]) and not np.array_equal(kc_got[:, rows], seed[:, rows])
    sess.close()
    for buf in const.values():
        if buf is not None:
            buf.free()
