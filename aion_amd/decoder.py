"""Synthetic decoder-only transformer assembled from the backend's steps (BASELINE config 5).

The step sequence is the one aion's graph compiler emits for a decoder (pattern of
src/bench/models.zig:433-536, trimmed to a plain pre-norm block): Gather -> per layer
[RMSNorm -> MatMul q,k,v -> RoPE1D(q,k) -> Cast f16 + SequenceAppend(k,v) -> Attention ->
MatMul o -> add -> RMSNorm -> MatMul gate,up -> gate(gelu) -> MatMul down -> add] ->
RMSNorm -> MatMul lm_head -> ArgMax. q4_0 weights are [K,N] quant_axis 0 MatMul operands (the
only q4 layout aion has), q8_0 weights are [N,K] quant_axis 1 MatMulNT operands.

Prefill runs the steps eagerly; the single-token decode step is recorded once into a program
(HIP graph) and replayed per token. Token id, position, cache write index and kv length stay in
device buffers: the argmax of one replay is the gather index of the next.
With `one_launch=True` (and a shape that qualifies) all blocks of a decode step run as ONE launch
(aionhip_step_decoder_stack); the step is then gather, that launch, the logits GEMV, the argmax and the
state advance. It gives the same bits as the recorded program; it is not the default because on MI355X it
measures 0.93 ms per token of the 26-layer decoder against 0.86 ms for the program replay.
"""
import math
from dataclasses import dataclass

import numpy as np

from . import backend as be


@dataclass
class DecoderConfig:
    layers: int = 26
    hidden: int = 2048
    heads: int = 8
    kv_heads: int = 1
    head_dim: int = 256
    ffn: int = 8192
    vocab: int = 262144
    max_seq: int = 256
    eps: float = 1e-6
    rope_base: float = 10000.0
    wdtype: int = be.Q4_0

    @property
    def q_dim(self):
        return self.heads * self.head_dim

    @property
    def kv_dim(self):
        return self.kv_heads * self.head_dim


def weight_shapes(cfg):
    """name -> (n, k) of every quantized matmul weight (C[.., n] = A[.., k] @ W)."""
    shapes = {}
    for l in range(cfg.layers):
        shapes["l%d.wq" % l] = (cfg.q_dim, cfg.hidden)
        shapes["l%d.wk" % l] = (cfg.kv_dim, cfg.hidden)
        shapes["l%d.wv" % l] = (cfg.kv_dim, cfg.hidden)
        shapes["l%d.wo" % l] = (cfg.hidden, cfg.q_dim)
        shapes["l%d.wgate" % l] = (cfg.ffn, cfg.hidden)
        shapes["l%d.wup" % l] = (cfg.ffn, cfg.hidden)
        shapes["l%d.wdown" % l] = (cfg.hidden, cfg.ffn)
    shapes["lm_head"] = (cfg.vocab, cfg.hidden)
    return shapes


class SyntheticWeights:
    """Seeded ~N(0,0.02) weights through the aion quantizers. A 2^22-sample normal pool is read at a
    per-tensor offset and tiled, which keeps a 2-billion-parameter model's set-up to seconds; the
    per-block statistics are those of N(0,0.02)."""

    def __init__(self, cfg, seed=0):
        self.cfg = cfg
        rng = np.random.default_rng(seed)
        self.pool = (rng.standard_normal(1 << 22) * 0.02).astype(np.float32)
        self.seed = seed

    def _values(self, name, count):
        off = (hash_name(name) * 2654435761 + self.seed) % (self.pool.size - 1)
        reps = -(-(count + off) // self.pool.size)
        return np.tile(self.pool, reps)[off:off + count]

    def blocks(self, name):
        n, k = weight_shapes(self.cfg)[name]
        v = self._values(name, n * k)
        if self.cfg.wdtype == be.Q8_0:
            return be.quantize_blocks(be.Q8_0, v.reshape(n, k), 1)       # [N,K] axis 1
        return be.quantize_blocks(be.Q4_0, v.reshape(k, n), 0)           # [K,N] axis 0

    def embed(self):
        return self._values("embed", self.cfg.vocab * self.cfg.hidden).reshape(self.cfg.vocab, self.cfg.hidden).copy()


def hash_name(name):
    h = 2166136261
    for ch in name.encode():
        h = ((h ^ ch) * 16777619) & 0xFFFFFFFF
    return h


class Decoder:
    def __init__(self, gpu, cfg, weights, on_weight=None, one_launch=False):
        """on_weight(name, host_array) is called for every tensor (the tests feed the oracle with it)."""
        self.gpu, self.cfg = gpu, cfg
        self.stack = None
        layout = be.ROWS_NK if cfg.wdtype == be.Q8_0 else be.KMAJOR_KN
        self.w = {}
        for name, (n, k) in weight_shapes(cfg).items():
            blocks = weights.blocks(name)
            self.w[name] = gpu.upload_weight(cfg.wdtype, layout, n, k, blocks)
            if on_weight:
                on_weight(name, blocks)
        emb = weights.embed()
        self.embed = gpu.upload(emb)
        if on_weight:
            on_weight("embed", emb)
        ones = np.ones(cfg.hidden, np.float32)
        self.gamma = gpu.upload(ones)          # every RMSNorm uses gamma = 1 (config 5)
        if on_weight:
            for l in range(cfg.layers):
                on_weight("l%d.norm1" % l, ones)
                on_weight("l%d.norm2" % l, ones)
            on_weight("norm_f", ones)
        kv_bytes = cfg.max_seq * cfg.kv_dim * 2
        self.kc = [gpu.zeros(kv_bytes) for _ in range(cfg.layers)]
        self.vc = [gpu.zeros(kv_bytes) for _ in range(cfg.layers)]
        self.one = gpu.upload(np.ones(1, np.int32))
        self.logits = gpu.alloc(cfg.vocab * 4)
        self.token = gpu.alloc(4)
        self.history = gpu.alloc(cfg.max_seq * 4)       # token produced at each position (decode program's log)
        self.state = {}        # S -> activation buffers
        self.program = None
        self.pos = 0
        if one_launch:
            layers = [{"wq": self.w["l%d.wq" % l], "wk": self.w["l%d.wk" % l], "wv": self.w["l%d.wv" % l], "wo": self.w["l%d.wo" % l],
                       "w_gate": self.w["l%d.wgate" % l], "w_up": self.w["l%d.wup" % l], "w_down": self.w["l%d.wdown" % l],
                       "norm1_gamma": self.gamma, "norm2_gamma": self.gamma, "k_cache": self.kc[l], "v_cache": self.vc[l]}
                      for l in range(cfg.layers)]
            try:
                self.stack = gpu.decoder_stack_create(layers, cfg.hidden, cfg.heads, cfg.kv_heads, cfg.head_dim, cfg.ffn, cfg.max_seq,
                                                      cfg.eps, cfg.eps, 1.0 / math.sqrt(cfg.head_dim), rope_base=cfg.rope_base)
            except be.AionHipError as e:
                if e.status != be.hip.UNSUPPORTED:
                    raise                                  # a shape outside the one-launch form's limits: separate steps

    def _buffers(self, s):
        if s in self.state:
            return self.state[s]
        c, g = self.cfg, self.gpu
        f = 4 * s
        b = {
            "ids": g.alloc(4 * s), "positions": g.alloc(4 * s), "write_index": g.alloc(4), "kv_len": g.alloc(4),
            "x": g.alloc(f * c.hidden), "h": g.alloc(f * c.hidden), "o": g.alloc(f * c.hidden),
            "q": g.alloc(f * c.q_dim), "qr": g.alloc(f * c.q_dim), "att": g.alloc(f * c.q_dim),
            "k": g.alloc(f * c.kv_dim), "kr": g.alloc(f * c.kv_dim), "v": g.alloc(f * c.kv_dim),
            "gate": g.alloc(f * c.ffn), "up": g.alloc(f * c.ffn), "act": g.alloc(f * c.ffn),
            "hl": g.alloc(4 * c.hidden),
        }
        self.state[s] = b
        return b

    def _forward(self, s, b):
        """Launches every step of one forward pass over `s` tokens (eagerly, or into an open recording)."""
        c, g = self.cfg, self.gpu
        g.step_gather_rows(be.F32, b["x"], self.embed, b["ids"], s, c.hidden, c.vocab)
        scale = 1.0 / math.sqrt(c.head_dim)
        for l in range(c.layers if not (s == 1 and self.stack is not None) else 0):
            p = "l%d." % l
            if s == 1 and c.hidden <= 8192 and c.head_dim % 8 == 0:
                # one new token: RMSNorm -> MatMul q, k, v -> RoPE1D(q), RoPE1D(k) -> f16 -> append, one launch
                g.step_rmsnorm_qkv_rope_append(self.w[p + "wq"], self.w[p + "wk"], self.w[p + "wv"], b["x"], self.gamma, c.eps,
                                               b["qr"], self.kc[l], self.vc[l], b["positions"], b["write_index"],
                                               c.max_seq, c.heads, c.kv_heads, c.head_dim, base=c.rope_base)
            else:
                # RMSNorm -> MatMul q, k, v (one call: the norm is not materialised)
                g.step_rmsnorm_matmul([self.w[p + "wq"], self.w[p + "wk"], self.w[p + "wv"]], b["x"], self.gamma, s,
                                      [b["q"], b["k"], b["v"]], c.eps)
                # RoPE1D(q), RoPE1D(k) -> f16 -> append, v -> f16 -> append
                g.step_rope_append(b["qr"], b["q"], b["k"], b["v"], self.kc[l], self.vc[l], b["positions"], b["write_index"],
                                   1, s, c.max_seq, c.heads, c.kv_heads, c.head_dim, base=c.rope_base)
            g.step_attention(b["att"], b["qr"], self.kc[l], self.vc[l], (1, s, c.max_seq, c.heads, c.kv_heads, c.head_dim, c.head_dim),
                             scale, q_dtype=be.F32, kv_dtype=be.F16, window=be.CAUSAL,
                             query_positions=b["positions"], kv_lengths=b["kv_len"])
            # MatMul o with beta = 1: x = x + att @ Wo (the residual add rides on the matmul's beta)
            g.step_matmul(self.w[p + "wo"], b["att"], s, b["x"], beta=1.0)
            if s == 1 and c.hidden <= 8192 and c.ffn % 32 == 0:
                # one row: RMSNorm -> MatMul gate, up -> gate(gelu) -> MatMul down (beta = 1), two launches
                g.step_rmsnorm_geglu_matmul(self.w[p + "wgate"], self.w[p + "wup"], self.w[p + "wdown"], b["x"], self.gamma, c.eps,
                                            b["x"], beta=1.0)
            else:
                g.step_rmsnorm_matmul([self.w[p + "wgate"], self.w[p + "wup"]], b["x"], self.gamma, s, [b["gate"], b["up"]], c.eps)
                # gate(gelu) -> MatMul down, beta = 1
                g.step_gate_matmul(self.w[p + "wdown"], b["gate"], b["up"], s, b["x"], beta=1.0)
        if s == 1 and self.stack is not None:
            g.step_decoder_stack(self.stack, b["x"], b["x"], b["positions"], b["write_index"], b["kv_len"])
        last = b["x"].view((s - 1) * c.hidden * 4)
        g.step_rmsnorm_matmul([self.w["lm_head"]], last, self.gamma, 1, [self.logits], c.eps)
        g.step_argmax(self.token, self.logits, 1, c.vocab)

    def reset(self):
        self.pos = 0

    def prefill(self, tokens):
        """Runs the prompt (positions pos .. pos+len-1); returns the greedy next token."""
        t = np.ascontiguousarray(tokens, np.int32)
        s = t.size
        if self.pos + s > self.cfg.max_seq:
            raise ValueError("prompt exceeds the cache capacity")
        b = self._buffers(s)
        g = self.gpu
        g.write(b["ids"], t)
        g.write(b["positions"], np.arange(self.pos, self.pos + s, dtype=np.int32))
        g.write(b["write_index"], np.array([self.pos], np.int32))
        g.write(b["kv_len"], np.array([self.pos + s], np.int32))
        self._forward(s, b)
        self.pos += s
        return int(g.download(self.token, np.int32, (1,))[0])

    def logits_host(self):
        return self.gpu.download(self.logits, np.float32, (self.cfg.vocab,))

    def begin_decode(self, first_token):
        """Prepares the single-token state and records the decode program (one warm-up step runs
        eagerly first so that every scratch buffer has its final size; it is then rolled back)."""
        g = self.gpu
        b = self._buffers(1)
        self._set_decode_state(b, first_token, self.pos)
        if self.program is not None and not g.program_is_current(self.program):
            # a longer prompt since the recording made the context replace a work buffer the program's launches address
            g.program_destroy(self.program)
            self.program = None
        if self.stack is not None:
            self._decode_buffers = b                 # one launch per step already: nothing to record
            return
        if self.program is None:
            self._forward(1, b)                      # eager warm-up at the current position
            g.sync()
            self._set_decode_state(b, first_token, self.pos)

            def issue():
                self._forward(1, b)
                # advance the device-resident loop state: next id = argmax, positions/write index/kv length += 1; the token
                # is also logged at the position it was produced at, so that a run of steps needs no read-back per step
                g.step_advance_state(b["ids"], self.token, 1, [b["positions"], b["write_index"], b["kv_len"]],
                                     log=self.history, log_index=b["positions"], log_capacity=self.cfg.max_seq)
            self.program = g.record_program(issue)

    def _set_decode_state(self, b, token, pos):
        g = self.gpu
        g.write(b["ids"], np.array([token], np.int32))
        g.write(b["positions"], np.array([pos], np.int32))
        g.write(b["write_index"], np.array([pos], np.int32))
        g.write(b["kv_len"], np.array([pos + 1], np.int32))

    def _step_on_device(self):
        """One decode step whose loop state stays on the device: the recorded program, or with the one-launch stack the five
        launches themselves."""
        if self.stack is None:
            self.gpu.program_execute(self.program)
            return
        b, g = self._decode_buffers, self.gpu
        self._forward(1, b)
        g.step_advance_state(b["ids"], self.token, 1, [b["positions"], b["write_index"], b["kv_len"]],
                             log=self.history, log_index=b["positions"], log_capacity=self.cfg.max_seq)

    def decode_step(self, read_token=True):
        """One decode step on the device-resident state; returns the token it produced (a 4-byte read-back)."""
        if self.pos + 1 > self.cfg.max_seq:
            raise ValueError("cache capacity exhausted")
        self._step_on_device()
        self.pos += 1
        if read_token:
            return int(self.gpu.download(self.token, np.int32, (1,))[0])
        return None

    def decode_run(self, n):
        """Replays the decode program n times back to back (nothing is read back in between: the loop state and the token
        log live on the device) and returns the n tokens."""
        if self.pos + n > self.cfg.max_seq:
            raise ValueError("cache capacity exhausted")
        start = self.pos
        for _ in range(n):
            self._step_on_device()
        self.pos += n
        tokens = self.gpu.download(self.history, np.int32, (n,), offset=start * 4)
        if self.stack is not None:
            self.gpu.decoder_stack_status(self.stack)      # raises if a launch gave up waiting (its tokens would be invalid)
        return tokens

    def decode_step_eager(self, token):
        """The same step without a program (used by tests to check the replayed graph)."""
        b = self._buffers(1)
        self._set_decode_state(b, token, self.pos)
        self._forward(1, b)
        self.pos += 1
        return int(self.gpu.download(self.token, np.int32, (1,))[0])

    def close(self):
        if self.program is not None:
            self.gpu.program_destroy(self.program)
            self.program = None
        if self.stack is not None:
            self.gpu.decoder_stack_destroy(self.stack)
            self.stack = None
        for w in self.w.values():
            w.free()
        for lst in (self.kc, self.vc):
            for t in lst:
                t.free()
        for bufs in self.state.values():
            for t in bufs.values():
                t.free()
        for t in (self.embed, self.gamma, self.one, self.logits, self.token, self.history):
            t.free()


class SessionDecoder:
    """The same decoder the way a compiled aion program reaches a backend: one record per step of the sequence in this
    module's header, nothing pre-fused, handed to the library's session executor (aionhip_session_execute), which folds
    what it may. Parameters are device tensors in aion's packed form; the session re-lays them at first use. The residual
    adds accumulate in place (x = x + o), the activations between the block's input and its output are workspace tensors.
    Gives the tokens of `Decoder` over the same weights."""

    def __init__(self, gpu, cfg, weights, fusion=None):
        from . import session as ss
        self.ss, self.gpu, self.cfg = ss, gpu, cfg
        self.sess = ss.Session(gpu)
        if fusion is not None:
            self.sess.set_fusion(fusion)
        self.nt = cfg.wdtype == be.Q8_0
        self.w = {name: gpu.upload(weights.blocks(name)) for name in weight_shapes(cfg)}
        self.embed = gpu.upload(weights.embed())
        self.gamma = gpu.upload(np.ones(cfg.hidden, np.float32))
        kv_bytes = cfg.max_seq * cfg.kv_dim * 2
        self.kc = [gpu.zeros(kv_bytes) for _ in range(cfg.layers)]
        self.vc = [gpu.zeros(kv_bytes) for _ in range(cfg.layers)]
        self.one = gpu.upload(np.ones(1, np.int32))
        self.logits = gpu.alloc(cfg.vocab * 4)
        self.token = gpu.alloc(4)
        self.state = {}
        self.program = None
        self.pos = 0

    def _weight(self, name):
        n, k = weight_shapes(self.cfg)[name]
        return self.ss.tensor(self.w[name], self.cfg.wdtype, (n, k) if self.nt else (k, n))

    def _program(self, s, advance=False):
        """-> (buffers, step records) of one forward pass over `s` tokens; advance: the loop state moves on the device
        behind it (the produced token becomes the next input, the three counters go up by one)."""
        key = (s, advance)
        if key in self.state:
            return self.state[key]
        c, g, ss = self.cfg, self.gpu, self.ss
        f4 = 4 * s
        b = self.state[(s, not advance)][0] if (s, not advance) in self.state else {
            "ids": g.alloc(4 * s), "positions": g.alloc(4 * s), "write_index": g.alloc(4), "kv_len": g.alloc(4),
            "x": g.alloc(f4 * c.hidden), "h": g.alloc(f4 * c.hidden), "o": g.alloc(f4 * c.hidden), "q": g.alloc(f4 * c.q_dim),
            "qr": g.alloc(f4 * c.q_dim), "att": g.alloc(f4 * c.q_dim), "k": g.alloc(f4 * c.kv_dim), "kr": g.alloc(f4 * c.kv_dim),
            "v": g.alloc(f4 * c.kv_dim), "k16": g.alloc(2 * s * c.kv_dim), "v16": g.alloc(2 * s * c.kv_dim), "gate": g.alloc(f4 * c.ffn),
            "up": g.alloc(f4 * c.ffn), "act": g.alloc(f4 * c.ffn), "hl": g.alloc(4 * c.hidden)}
        work = lambda nm, *shape: ss.tensor(b[nm], be.F32, shape, workspace=True)  # noqa: E731
        x = ss.tensor(b["x"], be.F32, (1, s, c.hidden))
        gamma = ss.tensor(self.gamma, be.F32, (c.hidden,))
        pos, widx, kvl = (ss.tensor(b[nm], be.I32, shape) for nm, shape in (("positions", (1, s)), ("write_index", (1,)), ("kv_len", (1,))))
        mm = (lambda p, a, w, out, **kw: p.matmul_nt(a, w, out, **kw)) if self.nt else (lambda p, a, w, out, **kw: p.matmul(a, w, out, **kw))
        p = ss.Steps()
        p.gather_rows(ss.tensor(self.embed, be.F32, (c.vocab, c.hidden)), ss.tensor(b["ids"], be.I32, (1, s)), x)
        for l in range(c.layers):
            n = "l%d." % l
            kc = ss.tensor(self.kc[l], be.F16, (1, c.max_seq, c.kv_heads, c.head_dim))
            vc = ss.tensor(self.vc[l], be.F16, (1, c.max_seq, c.kv_heads, c.head_dim))
            p.rmsnorm(x, gamma, None, work("h", 1, s, c.hidden), c.eps)
            mm(p, work("h", 1, s, c.hidden), self._weight(n + "wq"), work("q", 1, s, c.q_dim))
            mm(p, work("h", 1, s, c.hidden), self._weight(n + "wk"), work("k", 1, s, c.kv_dim))
            mm(p, work("h", 1, s, c.hidden), self._weight(n + "wv"), work("v", 1, s, c.kv_dim))
            p.rope1d(work("q", 1, s, c.heads, c.head_dim), pos, work("qr", 1, s, c.heads, c.head_dim), base_frequency=c.rope_base)
            p.rope1d(work("k", 1, s, c.kv_heads, c.head_dim), pos, work("kr", 1, s, c.kv_heads, c.head_dim), base_frequency=c.rope_base)
            k16 = ss.tensor(b["k16"], be.F16, (1, s, c.kv_heads, c.head_dim), workspace=True)
            v16 = ss.tensor(b["v16"], be.F16, (1, s, c.kv_heads, c.head_dim), workspace=True)
            p.cast(work("kr", 1, s, c.kv_heads, c.head_dim), k16)
            p.sequence_append(kc, k16, widx)
            p.cast(work("v", 1, s, c.kv_heads, c.head_dim), v16)
            p.sequence_append(vc, v16, widx)
            p.attention(work("qr", 1, s, c.heads, c.head_dim), kc, vc, work("att", 1, s, c.heads, c.head_dim), 1.0 / math.sqrt(c.head_dim),
                        query_positions=pos, kv_lengths=kvl)
            mm(p, work("att", 1, s, c.q_dim), self._weight(n + "wo"), work("o", 1, s, c.hidden))
            p.elemwise_binary(ss.ADD, x, work("o", 1, s, c.hidden), x)
            p.rmsnorm(x, gamma, None, work("h", 1, s, c.hidden), c.eps)
            mm(p, work("h", 1, s, c.hidden), self._weight(n + "wgate"), work("gate", 1, s, c.ffn))
            mm(p, work("h", 1, s, c.hidden), self._weight(n + "wup"), work("up", 1, s, c.ffn))
            p.elemwise_binary(ss.GATE, work("gate", 1, s, c.ffn), work("up", 1, s, c.ffn), work("act", 1, s, c.ffn), act=ss.GELU)
            mm(p, work("act", 1, s, c.ffn), self._weight(n + "wdown"), work("o", 1, s, c.hidden))
            p.elemwise_binary(ss.ADD, x, work("o", 1, s, c.hidden), x)
        last = ss.tensor(b["x"], be.F32, (1, c.hidden), offset=(s - 1) * c.hidden * 4)
        p.rmsnorm(last, gamma, None, work("hl", 1, c.hidden), c.eps)
        mm(p, work("hl", 1, c.hidden), self._weight("lm_head"), ss.tensor(self.logits, be.F32, (1, c.vocab)))
        p.argmax(ss.tensor(self.logits, be.F32, (1, c.vocab)), ss.tensor(self.token, be.I32, (1,)), axis=1)
        if advance:
            one = ss.tensor(self.one, be.I32, (1,))
            p.copy(ss.tensor(self.token, be.I32, (1,)), ss.tensor(b["ids"], be.I32, (1,)))
            for t in (pos, widx, kvl):
                p.elemwise_binary(ss.ADD, t, one, t)
        self.state[key] = (b, p, p.array())
        return self.state[key]

    def _set_state(self, b, tokens, pos):
        g, t = self.gpu, np.ascontiguousarray(tokens, np.int32)
        g.write(b["ids"], t)
        g.write(b["positions"], np.arange(pos, pos + t.size, dtype=np.int32))
        g.write(b["write_index"], np.array([pos], np.int32))
        g.write(b["kv_len"], np.array([pos + t.size], np.int32))

    def prefill(self, tokens):
        s = len(tokens)
        if self.pos + s > self.cfg.max_seq:
            raise ValueError("prompt exceeds the cache capacity")
        b, _, arr = self._program(s)
        self._set_state(b, tokens, self.pos)
        self.sess.execute(arr)
        self.pos += s
        return int(self.gpu.download(self.token, np.int32, (1,))[0])

    def logits_host(self):
        return self.gpu.download(self.logits, np.float32, (self.cfg.vocab,))

    def begin_decode(self, first_token):
        """One eager step at the current position (weights, scratch), rolled back, then the list recorded as a program."""
        g = self.gpu
        b, _, arr = self._program(1, advance=True)
        if self.program is not None and not g.program_is_current(self.program):
            g.program_destroy(self.program)
            self.program = None
        if self.program is None:
            self._set_state(b, [first_token], self.pos)
            self.sess.execute(arr)
            g.sync()
            self.calls_per_step = self.sess.stats()[0]
            self.program = g.record_program(lambda: self.sess.execute(arr))
        self._set_state(b, [first_token], self.pos)

    def decode_step(self, read_token=True):
        if self.pos + 1 > self.cfg.max_seq:
            raise ValueError("cache capacity exhausted")
        self.gpu.program_execute(self.program)
        self.pos += 1
        return int(self.gpu.download(self.token, np.int32, (1,))[0]) if read_token else None

    def close(self):
        if self.program is not None:
            self.gpu.program_destroy(self.program)
            self.program = None
        self.sess.close()
        for buf in list(self.w.values()) + [self.embed, self.gamma, self.one, self.logits, self.token] + self.kc + self.vc:
            buf.free()
        seen = set()
        for b, _, _ in self.state.values():
            for buf in b.values():
                if id(buf) not in seen:
                    seen.add(id(buf))
                    buf.free()
        self.state = {}
