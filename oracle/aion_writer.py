"""Writer for aion's package format (`.aion`, version 16) - TEST INFRASTRUCTURE ONLY (like everything under
oracle/): it makes the packages that the reader (`aion_amd/aion_file.py`) and the package runner are tested with.
Restates `src/aion/storage/aion_file/write.zig`: section order and offsets (write.zig:49-73), header and directory
(write.zig:607-623), tensor records with 64-byte aligned payloads (write.zig:204-239), and the per-op attribute
bytes that `parse.zig:485-640` reads back.

Parity: the reference holds no `.aion` file and no byte-level test of its writer, and its toolchain (Zig) is not
in this image, so nothing here is checked against bytes the reference produced: parity unpinned. What is checked:
the header / directory / strings / metadata layout against the reference's second statement of it
(`bindings/python/examples/_common.py:14-57`), and writer -> reader round trips.
"""
import struct

import numpy as np

DTYPES = {"f32": 0, "f16": 1, "i8": 2, "q4_0": 3, "q8_0": 4, "i32": 5}
BINARY_OPS = {n: i for i, n in enumerate(("add", "sub", "mul", "div", "eq", "ne", "lt", "gt", "le", "ge", "gate"))}
UNARY_OPS = {n: i for i, n in enumerate(("relu", "gelu", "silu", "sigmoid", "tanh", "sqrt", "log"))}
OPS = {n: i for i, n in enumerate((
    "MatMul", "ElemwiseBinary", "Unary", "Softmax", "Conv1D", "Conv2D", "LayerNorm", "RMSNorm", "Reduce", "Concat",
    "LSTMCell", "Copy", "ViewReshape", "ViewSqueeze", "ViewUnsqueeze", "ViewTranspose2D", "ViewSliceND", "RoPE1D",
    "SequenceAppend", "Attention", "Cast", "If", "Loop", "RFFT", "STFT", "RelPosMHA", "ArgMax", "ScatterRow",
    "Gather", "Dim", "Iota", "TopK", "MaxPool2D"))}
SECTION_IDS = {"strings": 1, "tensors": 2, "values": 3, "nodes": 4, "signatures": 5, "graph_meta": 6, "dim_symbols": 7,
               "dim_exprs": 8, "metadata": 9, "debug_names": 10, "regions": 11, "io_aliases": 12, "input_roles": 13}
ROLE_IDS = {"sequence_cache": 1, "cache_write_index": 2, "cache_visible_end": 3, "positions": 4, "tokens": 5, "state": 6}
INVALID = 0xFFFFFFFF
ALIGN = 64


def term(x):
    """A shape term: an int is a constant; ("expr", i) is dimension expression i. 16 bytes (write.zig, readShapeTerm)."""
    if isinstance(x, tuple):
        return struct.pack("<B7xQ", 1, x[1])
    return struct.pack("<B7xQ", 0, int(x))


def sym_attr(dims):
    return struct.pack("<I", len(dims)) + b"".join(term(d) for d in dims)


class PackageBuilder:
    """Collects the records of one package; `to_bytes()` lays the file out as write.zig:38-100 does."""

    def __init__(self):
        self.strings, self._string_ids = [], {}
        self.tensors, self.values, self.nodes = [], [], []
        self.inputs, self.outputs = [], []
        self.dim_symbols, self.dim_exprs = [], []
        self.metadata, self.debug_names, self.io_aliases, self.input_roles = [], [], [], []

    def string(self, s):
        if s not in self._string_ids:
            self._string_ids[s] = len(self.strings)
            self.strings.append(s)
        return self._string_ids[s]

    # ---- dimension symbols / expressions
    def symbol(self, name):
        """Adds a dimension symbol and the expression that names it; returns the ("expr", i) shape term."""
        self.dim_symbols.append(self.string(name))
        self.dim_exprs.append(struct.pack("<B3xI", 0, len(self.dim_symbols) - 1) + term(0) + term(0))
        return ("expr", len(self.dim_exprs) - 1)

    def expr(self, kind, lhs, rhs):
        code = {"add": 1, "sub": 2, "mul": 3, "floor_div": 4, "max": 5}[kind]
        self.dim_exprs.append(struct.pack("<B3xI", code, 0) + term(lhs) + term(rhs))
        return ("expr", len(self.dim_exprs) - 1)

    # ---- tensors and values
    def tensor_plain(self, dtype, array):
        data = np.ascontiguousarray(array).tobytes()
        self.tensors.append((struct.pack("<BBBBIIIiIQ", 0, DTYPES[dtype], 0, 0, INVALID, 1, 0, 0, 0, len(data)), b"", data))
        return len(self.tensors) - 1

    def tensor_quantized(self, scheme, blocks, quant_axis, logical_dtype="f32"):
        data = np.ascontiguousarray(blocks).tobytes()
        block_bytes = {"q8_0": 34, "q4_0": 18}[scheme]
        head = struct.pack("<BBBBIIIiIQ", 1, 0, DTYPES[logical_dtype], 0, self.string(scheme), 32, block_bytes, quant_axis, 0, len(data))
        self.tensors.append((head, b"", data))
        return len(self.tensors) - 1

    def value(self, dtype, shape, source="produced", initializer=None, name=None):
        src = {"input": 0, "initializer": 1, "produced": 2}[source]
        rec = struct.pack("<BBBBII", DTYPES[dtype], len(shape), src, 0, INVALID if initializer is None else initializer, len(shape))
        self.values.append(rec + b"".join(term(d) for d in shape))
        vid = len(self.values) - 1
        if name:
            self.debug_names.append((vid, self.string(name)))
        return vid

    def initializer(self, dtype, shape, tensor_index, name=None):
        return self.value(dtype, shape, "initializer", tensor_index, name)

    def input(self, name, dtype, shape, role=None, axis=0xFF, flags=1, capacity_symbol=INVALID, retained=0):
        vid = self.value(dtype, shape, "input", name=name)
        self.inputs.append((self.string(name), vid))
        if role:
            self.input_roles.append(struct.pack("<IBBBBII", len(self.inputs) - 1, ROLE_IDS[role], axis, flags, 0,
                                                capacity_symbol, retained))
        return vid

    def output(self, name, vid, alias_of_input=None):
        self.outputs.append((self.string(name), vid))
        if alias_of_input is not None:
            self.io_aliases.append((alias_of_input, len(self.outputs) - 1))

    # ---- nodes
    def node(self, op, inputs, out_dtype, out_shape, attrs=b"", name=None):
        out = self.value(out_dtype, out_shape, name=name)
        self.nodes.append(struct.pack("<HHIII", OPS[op], 0, out, len(inputs), len(attrs)) +
                          b"".join(struct.pack("<I", i) for i in inputs) + attrs)
        return out

    def matmul(self, a, b, shape, alpha=1.0, beta=0.0):
        return self.node("MatMul", (a, b), "f32", shape, struct.pack("<ff", alpha, beta))

    def binary(self, op, a, b, shape, dtype="f32"):
        return self.node("ElemwiseBinary", (a, b), dtype, shape, struct.pack("<B", BINARY_OPS[op]))

    def unary(self, op, a, shape):
        return self.node("Unary", (a,), "f32", shape, struct.pack("<B", UNARY_OPS[op]))

    def rmsnorm(self, x, gamma, beta, eps, shape, normalized):
        return self.node("RMSNorm", (x, gamma, beta), "f32", shape, struct.pack("<f", eps) + sym_attr(normalized))

    def reshape(self, x, dtype, shape):
        return self.node("ViewReshape", (x,), dtype, shape, sym_attr(shape))

    def transpose2d(self, x, dtype, shape):
        return self.node("ViewTranspose2D", (x,), dtype, shape)

    def rope(self, x, positions, shape, base, scale=1.0, proportion=1.0):
        return self.node("RoPE1D", (x, positions), "f32", shape, struct.pack("<fff", base, scale, proportion))

    def cast(self, x, to_dtype, shape):
        return self.node("Cast", (x,), to_dtype, shape, struct.pack("<B", DTYPES[to_dtype]))

    def sequence_append(self, cache, new, end_index, dtype, shape):
        return self.node("SequenceAppend", (cache, new, end_index), dtype, shape)

    def attention(self, q, k, v, positions, kv_lengths, shape, scale, window=(0xFFFFFFFF, 0, 0), soft_cap=0.0):
        ins = [q, k, v] + ([positions] if positions is not None else []) + ([kv_lengths] if kv_lengths is not None else [])
        controls = (1 if positions is not None else 0) | (2 if kv_lengths is not None else 0)
        return self.node("Attention", ins, "f32", shape, struct.pack("<fIIIfB", scale, window[0], window[1], window[2], soft_cap, controls))

    def gather(self, data, indices, shape, axis=0, batch_dims=0):
        return self.node("Gather", (data, indices), "f32", shape, struct.pack("<iQ", axis, batch_dims))

    def argmax(self, x, shape, axis=-1):
        return self.node("ArgMax", (x,), "i32", shape, struct.pack("<i", axis))

    # ---- file layout
    def _sections(self):
        u32 = lambda n: struct.pack("<I", n)
        strings = u32(len(self.strings)) + b"".join(u32(len(s.encode())) + s.encode() for s in self.strings)
        tensors = bytearray(u32(len(self.tensors)))
        for head, params, data in self.tensors:
            tensors += head + params
            tensors += b"\0" * (-len(tensors) % ALIGN)          # payload on a 64-byte offset of the section
            tensors += data
        named = lambda items: b"".join(struct.pack("<II", s, v) for s, v in items)
        meta_counts = (len(self.values), len(self.nodes), 0, len(self.tensors), len(self.inputs), len(self.outputs),
                       len(self.dim_symbols), len(self.dim_exprs), len(self.metadata), len(self.debug_names), len(self.io_aliases))
        out = [("strings", 1, strings), ("tensors", 1, bytes(tensors)),
               ("values", 1, u32(len(self.values)) + b"".join(self.values)),
               ("nodes", 1, u32(len(self.nodes)) + b"".join(self.nodes)),
               ("signatures", 1, struct.pack("<II", len(self.inputs), len(self.outputs)) + named(self.inputs) + named(self.outputs)),
               ("graph_meta", 1, struct.pack("<11I", *meta_counts))]
        if self.dim_symbols:
            out.append(("dim_symbols", 0, u32(len(self.dim_symbols)) + b"".join(u32(i) for i in self.dim_symbols)))
        if self.dim_exprs:
            out.append(("dim_exprs", 0, u32(len(self.dim_exprs)) + b"".join(self.dim_exprs)))
        if self.metadata:
            out.append(("metadata", 0, u32(len(self.metadata)) + named(self.metadata)))
        if self.debug_names:
            out.append(("debug_names", 0, u32(len(self.debug_names)) + named(self.debug_names)))
        if self.io_aliases:
            out.append(("io_aliases", 0, u32(len(self.io_aliases)) + named(self.io_aliases)))
        if self.input_roles:
            out.append(("input_roles", 0, u32(len(self.input_roles)) + b"".join(self.input_roles)))
        return out

    def add_metadata(self, key, value):
        self.metadata.append((self.string(key), self.string(value)))

    def to_bytes(self):
        # metadata strings are interned before the strings section is encoded
        sections = self._sections()
        dir_offset = 72
        at = dir_offset + 24 * len(sections)
        offsets = []
        for name, _flags, body in sections:
            if name == "tensors":
                at += -at % ALIGN
            offsets.append(at)
            at += len(body)
        total = at
        out = bytearray(b"AION" + struct.pack("<IIIQQQ", 16, len(sections), 0, dir_offset, total, 0) + b"\0" * 32)
        for (name, flags, body), off in zip(sections, offsets):
            out += struct.pack("<IIQQ", SECTION_IDS[name], flags, off, len(body))
        for (name, _flags, body), off in zip(sections, offsets):
            out += b"\0" * (off - len(out))
            out += body
        assert len(out) == total
        return bytes(out)


def build_decoder_package(cfg, blocks_of, embed, gammas=None, window=None, retained=0, growable=False):
    """The config-5 decoder authored as a graph (the pattern of src/bench/models.zig:433-536 trimmed to a plain
    pre-norm block; the weight and cache operands as aion declares them): inputs tokens [1,seq] i32, positions
    [1,seq] i32, write_index [1] i32, visible_end [1] i32, and per layer a k and a v cache [1,ctx,Hkv,D] f16 that
    alias the outputs of their SequenceAppend. Output 0 is the greedy token of the last position... as aion's
    ArgMax gives it: i32 [1,seq]; output 1 the logits [1,seq,vocab].

    cfg: layers, hidden, heads, kv_heads, head_dim, ffn, vocab, eps, rope_base, wdtype ("q4_0" | "q8_0");
    blocks_of(name) -> packed blocks ([K,N] quant_axis 0 for q4_0, [N,K] quant_axis 1 for q8_0); embed f32 [vocab,hidden].
    window: (left, right, chunk) of every Attention (default causal); retained > 0 declares the caches rolling rings
    that keep that many earlier positions (a sliding-window layer, src/bench/models.zig:440-447); growable sets the
    caches' allow_growable role flag."""
    b = PackageBuilder()
    seq, ctx = b.symbol("seq"), b.symbol("ctx")
    H, Hkv, D, E, F, V = cfg["heads"], cfg["kv_heads"], cfg["head_dim"], cfg["hidden"], cfg["ffn"], cfg["vocab"]
    q8 = cfg["wdtype"] == "q8_0"

    tokens = b.input("tokens", "i32", (1, seq), role="tokens", axis=1)
    positions = b.input("positions", "i32", (1, seq), role="positions", axis=1)
    write_index = b.input("write_index", "i32", (1,), role="cache_write_index")
    visible_end = b.input("visible_end", "i32", (1,), role="cache_visible_end")
    caches = []
    for l in range(cfg["layers"]):
        for kv in "kv":
            caches.append(b.input("l%d.%s_cache" % (l, kv), "f16", (1, ctx, Hkv, D), role="sequence_cache", axis=1,
                                  capacity_symbol=0 + 1, retained=retained,      # dim symbol 1 = "ctx"
                                  flags=3 if growable else 1))                  # zero_init | allow_growable (types.zig:179-183)

    def weight(name, k, n):
        blocks = blocks_of(name)
        if q8:      # [N,K] quant_axis 1, used through a transpose view (a file never holds MatMulNT: types.zig:19-21)
            t = b.tensor_quantized("q8_0", blocks, 1)
            w = b.initializer("q8_0", (n, k), t, name)
            return b.transpose2d(w, "q8_0", (k, n))
        t = b.tensor_quantized("q4_0", blocks, 0)
        return b.initializer("q4_0", (k, n), t, name)

    def vec(name, values):
        return b.initializer("f32", (len(values),), b.tensor_plain("f32", np.asarray(values, np.float32)), name)

    ones, zeros = np.ones(E, np.float32), np.zeros(E, np.float32)
    beta0 = vec("norm.beta", zeros)

    def rms(x, name, shape):
        g = vec(name, gammas[name] if gammas and name in gammas else ones)
        return b.rmsnorm(x, g, beta0, cfg["eps"], shape, (E,))

    table = b.initializer("f32", (V, E), b.tensor_plain("f32", embed), "embed")
    x = b.gather(table, tokens, (1, seq, E))
    for l in range(cfg["layers"]):
        p = "l%d." % l
        h = rms(x, p + "norm1", (1, seq, E))
        q = b.reshape(b.matmul(h, weight(p + "wq", E, H * D), (1, seq, H * D)), "f32", (1, seq, H, D))
        k = b.reshape(b.matmul(h, weight(p + "wk", E, Hkv * D), (1, seq, Hkv * D)), "f32", (1, seq, Hkv, D))
        v = b.reshape(b.matmul(h, weight(p + "wv", E, Hkv * D), (1, seq, Hkv * D)), "f32", (1, seq, Hkv, D))
        q = b.rope(q, positions, (1, seq, H, D), cfg["rope_base"])
        k = b.rope(k, positions, (1, seq, Hkv, D), cfg["rope_base"])
        kc = b.sequence_append(caches[2 * l], b.cast(k, "f16", (1, seq, Hkv, D)), write_index, "f16", (1, ctx, Hkv, D))
        vc = b.sequence_append(caches[2 * l + 1], b.cast(v, "f16", (1, seq, Hkv, D)), write_index, "f16", (1, ctx, Hkv, D))
        b.output("l%d.k_cache" % l, kc, alias_of_input=4 + 2 * l)
        b.output("l%d.v_cache" % l, vc, alias_of_input=4 + 2 * l + 1)
        o = b.attention(q, kc, vc, positions, visible_end, (1, seq, H, D), 1.0 / float(np.sqrt(D)),
                        window=window if window else (0xFFFFFFFF, 0, 0))
        o = b.matmul(b.reshape(o, "f32", (1, seq, H * D)), weight(p + "wo", H * D, E), (1, seq, E))
        x = b.binary("add", x, o, (1, seq, E))
        h = rms(x, p + "norm2", (1, seq, E))
        gate = b.matmul(h, weight(p + "wgate", E, F), (1, seq, F))
        up = b.matmul(h, weight(p + "wup", E, F), (1, seq, F))
        act = b.binary("mul", b.unary("gelu", gate, (1, seq, F)), up, (1, seq, F))
        x = b.binary("add", x, b.matmul(act, weight(p + "wdown", F, E), (1, seq, E)), (1, seq, E))
    h = rms(x, "norm_f", (1, seq, E))
    logits = b.matmul(h, weight("lm_head", E, V), (1, seq, V))
    token = b.argmax(logits, (1, seq))
    # the signature lists the token first; the caches were added as outputs while the layers were built
    b.outputs.insert(0, (b.string("next_token"), token))
    b.outputs.insert(1, (b.string("logits"), logits))
    b.io_aliases = [(i, o + 2) for i, o in b.io_aliases]
    b.add_metadata("arch", "synthetic-decoder")
    b.add_metadata("layers", str(cfg["layers"]))
    return b.to_bytes()


def build_sandwich_decoder_package(cfg, blocks_of, table_blocks, gammas):
    """A decoder in the shape of aion's own bench model (src/bench/models.zig:433-536, without its per-layer-input
    branch and kv sharing): a tied, block-quantized embedding table that is gathered from AND contracted against
    (through a ViewTranspose2D) for the logits; the embedding scaled by sqrt(hidden); per-head RMSNorm on q, k and v;
    attention with scale 1; RMSNorm on the attention and feed-forward outputs before their residual adds; local layers
    with a sliding window over rolling caches of `local_window` rows (window left = local_window - 1, that many
    positions retained: models.zig:66-68, 301-310, 440-445) and every `global_every`-th layer global over [1,ctx,..]
    caches with its own RoPE base; logits soft-capped as scale * tanh(logits / scale) before the ArgMax.

    cfg: layers, hidden, heads, kv_heads, head_dim, ffn, vocab, eps, rope_base_local, rope_base_global, local_window,
    global_every, logit_softcap, wdtype. blocks_of(name) as in build_decoder_package; table_blocks: the embedding
    table [vocab, hidden] as q8_0 blocks along its rows (quant_axis 1); gammas: name -> f32 vector for every norm
    ("l%d.norm_in", "l%d.q_norm", "l%d.k_norm", "l%d.v_norm", "l%d.norm_attn", "l%d.norm_ffn_in", "l%d.norm_ffn", "norm_f")."""
    b = PackageBuilder()
    seq, ctx = b.symbol("seq"), b.symbol("ctx")
    H, Hkv, D, E, F, V = cfg["heads"], cfg["kv_heads"], cfg["head_dim"], cfg["hidden"], cfg["ffn"], cfg["vocab"]
    W = cfg["local_window"]
    q8 = cfg["wdtype"] == "q8_0"
    is_global = lambda l: l % cfg["global_every"] == cfg["global_every"] - 1

    tokens = b.input("tokens", "i32", (1, seq), role="tokens", axis=1)
    positions = b.input("positions", "i32", (1, seq), role="positions", axis=1)
    write_index = b.input("write_index", "i32", (1,), role="cache_write_index")
    visible_end = b.input("visible_end", "i32", (1,), role="cache_visible_end")
    caches = []
    for l in range(cfg["layers"]):
        for kv in "kv":
            if is_global(l):
                caches.append(b.input("l%d.%s_cache" % (l, kv), "f16", (1, ctx, Hkv, D), role="sequence_cache", axis=1, capacity_symbol=1))
            else:
                caches.append(b.input("l%d.%s_cache" % (l, kv), "f16", (1, W, Hkv, D), role="sequence_cache", axis=1, retained=W - 1))

    def weight(name, k, n):
        blocks = blocks_of(name)
        if q8:
            w = b.initializer("q8_0", (n, k), b.tensor_quantized("q8_0", blocks, 1), name)
            return b.transpose2d(w, "q8_0", (k, n))
        return b.initializer("q4_0", (k, n), b.tensor_quantized("q4_0", blocks, 0), name)

    def vec(name, values):
        return b.initializer("f32", (len(values),), b.tensor_plain("f32", np.asarray(values, np.float32)), name)

    def scalar(value):
        return b.initializer("f32", (1,), b.tensor_plain("f32", np.asarray([value], np.float32)))

    betas = {n: vec("beta%d" % n, np.zeros(n, np.float32)) for n in (E, D)}

    def rms(x, name, shape):
        n = shape[-1]
        return b.rmsnorm(x, vec(name, gammas[name]), betas[n], cfg["eps"], shape, (n,))

    table = b.initializer("q8_0", (V, E), b.tensor_quantized("q8_0", table_blocks, 1), "embed")
    x = b.binary("mul", b.gather(table, tokens, (1, seq, E)), scalar(float(np.sqrt(np.float32(E)))), (1, seq, E))
    for l in range(cfg["layers"]):
        p = "l%d." % l
        base = cfg["rope_base_global"] if is_global(l) else cfg["rope_base_local"]
        t_len = ctx if is_global(l) else W
        h = rms(x, p + "norm_in", (1, seq, E))
        q = b.reshape(b.matmul(h, weight(p + "wq", E, H * D), (1, seq, H * D)), "f32", (1, seq, H, D))
        q = b.rope(rms(q, p + "q_norm", (1, seq, H, D)), positions, (1, seq, H, D), base)
        k = b.reshape(b.matmul(h, weight(p + "wk", E, Hkv * D), (1, seq, Hkv * D)), "f32", (1, seq, Hkv, D))
        k = b.rope(rms(k, p + "k_norm", (1, seq, Hkv, D)), positions, (1, seq, Hkv, D), base)
        v = b.reshape(b.matmul(h, weight(p + "wv", E, Hkv * D), (1, seq, Hkv * D)), "f32", (1, seq, Hkv, D))
        v = rms(v, p + "v_norm", (1, seq, Hkv, D))
        kc = b.sequence_append(caches[2 * l], b.cast(k, "f16", (1, seq, Hkv, D)), write_index, "f16", (1, t_len, Hkv, D))
        vc = b.sequence_append(caches[2 * l + 1], b.cast(v, "f16", (1, seq, Hkv, D)), write_index, "f16", (1, t_len, Hkv, D))
        b.output("l%d.k_cache" % l, kc, alias_of_input=4 + 2 * l)
        b.output("l%d.v_cache" % l, vc, alias_of_input=4 + 2 * l + 1)
        window = (0xFFFFFFFF, 0, 0) if is_global(l) else (W - 1, 0, 0)
        o = b.attention(q, kc, vc, positions, visible_end, (1, seq, H, D), 1.0, window=window)
        o = b.matmul(b.reshape(o, "f32", (1, seq, H * D)), weight(p + "wo", H * D, E), (1, seq, E))
        x = b.binary("add", x, rms(o, p + "norm_attn", (1, seq, E)), (1, seq, E))
        h = rms(x, p + "norm_ffn_in", (1, seq, E))
        gate = b.matmul(h, weight(p + "wgate", E, F), (1, seq, F))
        up = b.matmul(h, weight(p + "wup", E, F), (1, seq, F))
        act = b.binary("mul", b.unary("gelu", gate, (1, seq, F)), up, (1, seq, F))
        ff = b.matmul(act, weight(p + "wdown", F, E), (1, seq, E))
        x = b.binary("add", x, rms(ff, p + "norm_ffn", (1, seq, E)), (1, seq, E))
    h = rms(x, "norm_f", (1, seq, E))
    logits = b.matmul(h, b.transpose2d(table, "q8_0", (E, V)), (1, seq, V))
    cap = cfg["logit_softcap"]
    capped = b.binary("mul", b.unary("tanh", b.binary("mul", logits, scalar(1.0 / cap), (1, seq, V)), (1, seq, V)), scalar(cap), (1, seq, V))
    token = b.argmax(capped, (1, seq))
    b.outputs.insert(0, (b.string("next_token"), token))
    b.outputs.insert(1, (b.string("logits"), capped))
    b.io_aliases = [(i, o + 2) for i, o in b.io_aliases]
    b.add_metadata("arch", "synthetic-sandwich-decoder")
    b.add_metadata("layers", str(cfg["layers"]))
    return b.to_bytes()
