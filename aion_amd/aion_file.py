"""Reader for aion's model package format (`.aion`, version 16): the data format on the caller's side of
the backend. Restates `src/aion/storage/aion_file/parse.zig` (records) and `types.zig` (constants, enums);
every function cites the lines it follows. Little-endian throughout.

Layout (parse.zig:59-69, 175-196): a 72-byte header (magic "AION", u32 version = 16, u32 section count, u32
reserved, u64 directory offset, u64 file size, u64 flags, 32 reserved bytes), a directory of 24-byte entries
(u32 type, u32 flags with bit 0 = required, u64 offset, u64 size), then the sections. Tensor payloads start on
64-byte file offsets (types.zig:24-26) and are returned as views of the mapped file, never copied.

What pins this reader: header, directory, strings and metadata are stated a second time by the reference's own
Python example (`bindings/python/examples/_common.py:14-57`); the tensor, value and node records have no fixture
in the reference (it holds no `.aion` file and no byte-level test), so for those this reader is checked only
against the writer in `oracle/aion_writer.py`, written from `write.zig`: parity unpinned.
"""
import mmap
import struct
from dataclasses import dataclass, field

import numpy as np

MAGIC = b"AION"
VERSION = 16                      # types.zig:22
PAYLOAD_ALIGNMENT = 64            # types.zig:26
HEADER_SIZE = 72                  # types.zig:27
SECTION_DESC_SIZE = 24            # types.zig:28
INVALID_INDEX = 0xFFFFFFFF        # types.zig:29

# types.zig:40-54
SECTIONS = {1: "strings", 2: "tensors", 3: "values", 4: "nodes", 5: "signatures", 6: "graph_meta", 7: "dim_symbols",
            8: "dim_exprs", 9: "metadata", 10: "debug_names", 11: "regions", 12: "io_aliases", 13: "input_roles"}
REQUIRED = ("strings", "tensors", "values", "nodes", "signatures", "graph_meta")

# backend/types.zig:29-38, 92-109, 119-127
DTYPES = ("f32", "f16", "i8", "q4_0", "q8_0", "i32")
BINARY_OPS = ("add", "sub", "mul", "div", "eq", "ne", "lt", "gt", "le", "ge", "gate")
UNARY_OPS = ("relu", "gelu", "silu", "sigmoid", "tanh", "sqrt", "log")
REDUCE_OPS = ("sum", "mean")
PAD_MODES = ("zero", "reflect")
VALUE_SOURCES = ("input", "initializer", "produced")              # types.zig:127-131
# graph/graph.zig:62-128
OPS = ("MatMul", "ElemwiseBinary", "Unary", "Softmax", "Conv1D", "Conv2D", "LayerNorm", "RMSNorm", "Reduce", "Concat",
       "LSTMCell", "Copy", "ViewReshape", "ViewSqueeze", "ViewUnsqueeze", "ViewTranspose2D", "ViewSliceND", "RoPE1D",
       "SequenceAppend", "Attention", "Cast", "If", "Loop", "RFFT", "STFT", "RelPosMHA", "ArgMax", "ScatterRow",
       "Gather", "Dim", "Iota", "TopK", "MaxPool2D")
# types.zig:164-177
INPUT_ROLES = {1: "sequence_cache", 2: "cache_write_index", 3: "cache_visible_end", 4: "positions", 5: "tokens", 6: "state"}
DIM_EXPR_KINDS = ("symbol", "add", "sub", "mul", "floor_div", "max")   # parse.zig:312-320


class PackageError(ValueError):
    """kind is one of the reference's PackageError names (types.zig:31-38)."""

    def __init__(self, kind, message):
        super().__init__("%s: %s" % (kind, message))
        self.kind = kind


@dataclass
class Tensor:
    """One initializer (parse.zig:329-381). `data` is a uint8 view of the file."""
    quantized: bool
    dtype: str                      # plain: the scalar dtype; quantized: the logical dtype
    scheme: str = ""                # "q8_0" / "q4_0" for quantized tensors
    block_elems: int = 1
    block_bytes: int = 0
    quant_axis: int = 0
    params: bytes = b""
    data: np.ndarray = None


@dataclass
class Value:
    """parse.zig:383-408. shape: one term per axis, ("const", n) or ("expr", dim-expression index)."""
    dtype: str
    rank: int
    source: str
    initializer: int = None
    shape: tuple = ()


@dataclass
class Node:
    """parse.zig:410-439; attrs per parse.zig:485-640."""
    op: str
    output: int
    inputs: tuple
    attrs: dict = field(default_factory=dict)
    extra_outputs: tuple = ()


@dataclass
class InputRole:
    """parse.zig:722-748, types.zig:164-198."""
    input: int
    kind: str
    axis: int
    flags: int
    capacity_symbol: int
    retained_history_tokens: int


@dataclass
class Package:
    strings: list
    tensors: list
    values: list
    nodes: list
    regions: list
    inputs: list                    # (name, value id)
    outputs: list
    graph_meta: dict
    dim_symbols: list
    dim_exprs: list                 # (kind, aux, lhs term, rhs term)
    metadata: dict
    debug_names: dict               # value id -> name
    io_aliases: list                # (input index, output index)
    input_roles: list
    _mapping: object = None

    def dim_term(self, term, symbols):
        """Size of one shape term under `symbols` (name -> int); parse.zig:291-327 for the expression kinds."""
        kind, payload = term
        if kind == "const":
            return int(payload)
        ekind, aux, lhs, rhs = self.dim_exprs[payload]
        if ekind == "symbol":
            name = self.dim_symbols[aux]
            if name not in symbols:
                raise PackageError("InvalidArgument", "dimension symbol %r is unbound" % name)
            return int(symbols[name])
        a, b = self.dim_term(lhs, symbols), self.dim_term(rhs, symbols)
        if ekind == "add":
            return a + b
        if ekind == "sub":
            return a - b
        if ekind == "mul":
            return a * b
        if ekind == "floor_div":
            return a // b
        return max(a, b)

    def shape_of(self, value_id, symbols):
        return tuple(self.dim_term(t, symbols) for t in self.values[value_id].shape)

    def role_of_input(self, input_index):
        for r in self.input_roles:
            if r.input == input_index:
                return r
        return None


class _Cursor:
    """parse.zig:838-870 (readBytes / readIntCursor): every read is bounds-checked against the section."""

    def __init__(self, buf, what):
        self.buf, self.pos, self.what = buf, 0, what

    def take(self, n):
        if n < 0 or self.pos + n > len(self.buf):
            raise PackageError("InvalidFormat", "%s: truncated (need %d bytes at %d of %d)" % (self.what, n, self.pos, len(self.buf)))
        out = self.buf[self.pos:self.pos + n]
        self.pos += n
        return out

    def unpack(self, fmt):
        return struct.unpack("<" + fmt, bytes(self.take(struct.calcsize("<" + fmt))))

    def u8(self):
        return self.unpack("B")[0]

    def u16(self):
        return self.unpack("H")[0]

    def u32(self):
        return self.unpack("I")[0]

    def i32(self):
        return self.unpack("i")[0]

    def u64(self):
        return self.unpack("Q")[0]

    def f32(self):
        return self.unpack("f")[0]

    def enum(self, names):
        raw = self.u8()
        if raw >= len(names):
            raise PackageError("InvalidFormat", "%s: enum code %d" % (self.what, raw))
        return names[raw]

    def done(self):
        if self.pos != len(self.buf):
            raise PackageError("InvalidFormat", "%s: %d trailing bytes" % (self.what, len(self.buf) - self.pos))


def _shape_term(c):
    """parse.zig:827-836: u8 kind, 7 pad bytes, u64 payload."""
    kind = c.u8()
    c.take(7)
    payload = c.u64()
    if kind == 0:
        return ("const", payload)
    if kind == 1:
        if payload > 0xFFFFFFFF:
            raise PackageError("InvalidFormat", "dimension expression index out of range")
        return ("expr", payload)
    raise PackageError("InvalidFormat", "shape term kind %d" % kind)


def _sym_attr(c):
    """parse.zig:775-804: u32 count, count shape terms."""
    return tuple(_shape_term(c) for _ in range(c.u32()))


def _window(c):
    return {"left": c.u32(), "right": c.u32(), "chunk": c.u32()}     # parse.zig:806-812


def _strings(buf):
    """parse.zig:272-284. aion keeps strings as raw bytes without validating them; bytes that are not UTF-8 survive here
    as surrogate escapes (`s.encode("utf-8", "surrogateescape")` gives them back) instead of failing the parse."""
    c = _Cursor(buf, "strings")
    out = []
    for _ in range(c.u32()):
        out.append(bytes(c.take(c.u32())).decode("utf-8", "surrogateescape"))
    c.done()
    return out


def _string_index(c, strings):
    idx = c.u32()
    if idx >= len(strings):
        raise PackageError("InvalidFormat", "%s: string index %d of %d" % (c.what, idx, len(strings)))
    return idx


def _tensors(buf, strings):
    """parse.zig:329-381. The payload of every tensor starts on a 64-byte offset of the section, which itself
    starts on one (checked by the caller)."""
    c = _Cursor(buf, "tensors")
    out = []
    for _ in range(c.u32()):
        kind, plain_raw, logical_raw, _pad = c.unpack("BBBB")
        scheme_idx, block_elems, block_bytes = c.unpack("III")
        quant_axis = c.i32()
        params_len = c.u32()
        data_len = c.u64()
        params = bytes(c.take(params_len))
        c.take(-c.pos % PAYLOAD_ALIGNMENT)
        data = np.frombuffer(c.take(data_len), dtype=np.uint8)
        if kind == 0:
            if plain_raw >= len(DTYPES):
                raise PackageError("InvalidFormat", "tensor dtype %d" % plain_raw)
            out.append(Tensor(False, DTYPES[plain_raw], data=data))
        elif kind == 1:
            if scheme_idx == INVALID_INDEX or scheme_idx >= len(strings) or logical_raw >= len(DTYPES):
                raise PackageError("InvalidFormat", "quantized tensor without a scheme")
            out.append(Tensor(True, DTYPES[logical_raw], strings[scheme_idx], block_elems, block_bytes, quant_axis, params, data))
        else:
            raise PackageError("InvalidFormat", "tensor kind %d" % kind)
    c.done()
    return out


def _values(buf):
    """parse.zig:383-408."""
    c = _Cursor(buf, "values")
    out = []
    for _ in range(c.u32()):
        dtype = c.enum(DTYPES)
        rank = c.u8()
        source = c.enum(VALUE_SOURCES)
        c.u8()
        init = c.u32()
        terms = tuple(_shape_term(c) for _ in range(c.u32()))
        out.append(Value(dtype, rank, source, None if init == INVALID_INDEX else init, terms))
    c.done()
    return out


def _node_attrs(op, buf):
    """parse.zig:485-640: the attribute bytes of one node; they must be consumed exactly."""
    c = _Cursor(buf, "attrs of " + op)
    a, extra = {}, ()
    size = c.u64
    if op == "MatMul":
        a = {"alpha": c.f32(), "beta": c.f32()}
    elif op == "ElemwiseBinary":
        a = {"op": c.enum(BINARY_OPS)}
    elif op == "Unary":
        a = {"op": c.enum(UNARY_OPS)}
    elif op in ("Softmax", "Concat", "ArgMax", "Dim", "Iota", "ViewUnsqueeze"):
        a = {"axis": c.i32()}
    elif op == "If":
        a = {"then_region": c.u32(), "else_region": c.u32()}
    elif op == "Loop":
        a = {"body_region": c.u32(), "static_max_trip_count": size()}
        cond = c.i32()
        a["cond_carry"] = None if cond < 0 else cond
        a["check_before"] = c.u8() != 0
        extra = tuple(c.u32() for _ in range(c.u32()))
    elif op == "TopK":
        a = {"k": size(), "axis": c.i32(), "largest": c.u8() != 0}
        n_extra = c.u32()
        if n_extra != 1:
            raise PackageError("InvalidFormat", "TopK with %d extra outputs" % n_extra)
        extra = (c.u32(),)
    elif op == "Conv1D":
        a = {"stride": size(), "dilation": size(), "pad_left": size(), "pad_right": size(), "pad_mode": c.enum(PAD_MODES), "groups": size()}
    elif op == "MaxPool2D":
        for k in ("kernel_h", "kernel_w", "stride_h", "stride_w", "dilation_h", "dilation_w", "pad_top", "pad_bottom", "pad_left", "pad_right"):
            a[k] = size()
        ceil_raw = c.u8()
        if ceil_raw > 1:
            raise PackageError("InvalidFormat", "MaxPool2D ceil_mode %d" % ceil_raw)
        a["ceil_mode"] = ceil_raw != 0
    elif op == "Conv2D":
        for k in ("stride_h", "stride_w", "dilation_h", "dilation_w", "pad_top", "pad_bottom", "pad_left", "pad_right"):
            a[k] = size()
        a["pad_mode"] = c.enum(PAD_MODES)
        a["groups"] = size()
    elif op in ("LayerNorm", "RMSNorm"):
        a = {"eps": c.f32(), "normalized_shape": _sym_attr(c)}
    elif op == "Attention":
        a = {"scale": c.f32(), "window": _window(c), "soft_cap": c.f32()}
        controls = c.u8()
        if controls & ~3:
            raise PackageError("InvalidFormat", "Attention controls %#x" % controls)
        a["has_query_positions"], a["has_kv_lengths"] = bool(controls & 1), bool(controls & 2)
    elif op == "Reduce":
        a = {"op": c.enum(REDUCE_OPS)}
        a["axis"] = c.i32() if c.u8() else None
    elif op == "LSTMCell":
        a = {"has_bias": c.u8() != 0}
    elif op == "STFT":
        a = {"n_fft": size(), "hop_length": size(), "center": c.u8() != 0}
    elif op == "RelPosMHA":
        a = {"scale": c.f32(), "has_mask": c.u8() != 0, "window": _window(c), "relative_zero_index": size(), "soft_cap": c.f32()}
    elif op == "Gather":
        a = {"axis": c.i32(), "batch_dims": size()}
    elif op == "RoPE1D":
        a = {"base_frequency": c.f32(), "scale_factor": c.f32(), "rope_proportion": c.f32()}
    elif op == "Cast":
        a = {"to_dtype": c.enum(DTYPES)}
    elif op == "ViewReshape":
        a = {"new_shape": _sym_attr(c)}
    elif op == "ViewSqueeze":
        a = {"axis": c.i32() if c.u8() else None}
    elif op == "ViewSliceND":
        a = {"starts": tuple(size() for _ in range(c.u32())), "lens": _sym_attr(c)}
    elif op in ("RFFT", "ScatterRow", "Copy", "SequenceAppend", "ViewTranspose2D"):
        pass
    else:
        raise PackageError("InvalidFormat", "operation %r" % op)
    c.done()
    return a, extra


def _node_records(c):
    """parse.zig:410-439: u16 op, u16 zero, u32 output, u32 input count, u32 attribute length, inputs, attributes."""
    out = []
    for _ in range(c.u32()):
        op_raw = c.u16()
        if c.u16() != 0:
            raise PackageError("InvalidFormat", "node reserved field")
        output, n_inputs, attr_len = c.unpack("III")
        inputs = tuple(c.u32() for _ in range(n_inputs))
        attr = c.take(attr_len)
        if op_raw >= len(OPS):
            raise PackageError("InvalidFormat", "operation tag %d" % op_raw)
        attrs, extra = _node_attrs(OPS[op_raw], attr)
        out.append(Node(OPS[op_raw], output, inputs, attrs, extra))
    return out


def _nodes(buf):
    c = _Cursor(buf, "nodes")
    out = _node_records(c)
    c.done()
    return out


def _regions(buf):
    """parse.zig:451-479: per region a node list and its output value ids."""
    c = _Cursor(buf, "regions")
    out = []
    for _ in range(c.u32()):
        nodes = _node_records(c)
        out.append((nodes, tuple(c.u32() for _ in range(c.u32()))))
    c.done()
    return out


def _signatures(buf, strings):
    """parse.zig:642-671."""
    c = _Cursor(buf, "signatures")
    n_in, n_out = c.u32(), c.u32()
    named = lambda: (strings[_string_index(c, strings)], c.u32())
    ins = [named() for _ in range(n_in)]
    outs = [named() for _ in range(n_out)]
    c.done()
    return ins, outs


def _graph_meta(buf):
    """parse.zig:750-767: eleven u32 counts."""
    c = _Cursor(buf, "graph_meta")
    keys = ("values", "nodes", "regions", "initializers", "inputs", "outputs", "dim_symbols", "dim_exprs", "metadata", "debug_names", "io_aliases")
    out = {k: c.u32() for k in keys}
    c.done()
    return out


def _dim_symbols(buf, strings):
    c = _Cursor(buf, "dim_symbols")                                # parse.zig:291-302
    out = [strings[_string_index(c, strings)] for _ in range(c.u32())]
    c.done()
    return out


def _dim_exprs(buf):
    c = _Cursor(buf, "dim_exprs")                                  # parse.zig:304-327
    out = []
    for _ in range(c.u32()):
        kind = c.enum(DIM_EXPR_KINDS)
        c.take(3)
        aux = c.u32()
        out.append((kind, aux, _shape_term(c), _shape_term(c)))
    c.done()
    return out


def _metadata(buf, strings):
    c = _Cursor(buf, "metadata")                                   # parse.zig:673-688
    out = {}
    for _ in range(c.u32()):
        k = strings[_string_index(c, strings)]
        out[k] = strings[_string_index(c, strings)]
    c.done()
    return out


def _debug_names(buf, strings):
    c = _Cursor(buf, "debug_names")                                # parse.zig:690-705
    out = {}
    for _ in range(c.u32()):
        value = c.u32()
        out[value] = strings[_string_index(c, strings)]
    c.done()
    return out


def _io_aliases(buf):
    c = _Cursor(buf, "io_aliases")                                 # parse.zig:707-720
    out = [(c.u32(), c.u32()) for _ in range(c.u32())]
    c.done()
    return out


def _input_roles(buf):
    c = _Cursor(buf, "input_roles")                                # parse.zig:722-748
    out = []
    for _ in range(c.u32()):
        inp = c.u32()
        kind_raw, axis, flags, reserved = c.unpack("BBBB")
        cap, retained = c.u32(), c.u32()
        if reserved != 0 or kind_raw not in INPUT_ROLES:
            raise PackageError("InvalidFormat", "input role record")
        out.append(InputRole(inp, INPUT_ROLES[kind_raw], axis, flags, cap, retained))
    c.done()
    return out


def parse(buf):
    """Parses a whole package from a bytes-like object (parse.zig:46-161)."""
    view = memoryview(buf).cast("B")
    if len(view) < HEADER_SIZE or bytes(view[:4]) != MAGIC:
        raise PackageError("InvalidFormat", "not an aion package")
    version, n_sections, _reserved = struct.unpack_from("<III", view, 4)
    if version != VERSION:
        raise PackageError("UnsupportedVersion", "version %d (only %d is read)" % (version, VERSION))
    dir_offset, file_size, _flags = struct.unpack_from("<QQQ", view, 16)
    if file_size != len(view):
        raise PackageError("InvalidFormat", "header says %d bytes, the file has %d" % (file_size, len(view)))
    refs = {}
    if dir_offset + n_sections * SECTION_DESC_SIZE > len(view):
        raise PackageError("InvalidFormat", "section directory outside the file")
    for i in range(n_sections):
        stype, flags, off, size = struct.unpack_from("<IIQQ", view, dir_offset + i * SECTION_DESC_SIZE)
        if off + size > len(view):
            raise PackageError("InvalidFormat", "section %d outside the file" % stype)
        if stype not in SECTIONS:
            if flags & 1:
                raise PackageError("UnsupportedFeature", "unknown required section type %d" % stype)
            continue
        name = SECTIONS[stype]
        if name in refs:
            raise PackageError("InvalidFormat", "section %s twice" % name)
        refs[name] = (flags, off, size)
    for name in REQUIRED:
        if name not in refs or not refs[name][0] & 1:
            raise PackageError("InvalidFormat", "required section %s is missing" % name)
    sec = lambda name: view[refs[name][1]:refs[name][1] + refs[name][2]]
    strings = _strings(sec("strings"))
    if refs["tensors"][1] % PAYLOAD_ALIGNMENT:
        raise PackageError("InvalidFormat", "the tensors section does not start on a 64-byte offset")
    ins, outs = _signatures(sec("signatures"), strings)
    pkg = Package(
        strings=strings,
        tensors=_tensors(sec("tensors"), strings),
        values=_values(sec("values")),
        nodes=_nodes(sec("nodes")),
        regions=_regions(sec("regions")) if "regions" in refs else [],
        inputs=ins, outputs=outs,
        graph_meta=_graph_meta(sec("graph_meta")),
        dim_symbols=_dim_symbols(sec("dim_symbols"), strings) if "dim_symbols" in refs else [],
        dim_exprs=_dim_exprs(sec("dim_exprs")) if "dim_exprs" in refs else [],
        metadata=_metadata(sec("metadata"), strings) if "metadata" in refs else {},
        debug_names=_debug_names(sec("debug_names"), strings) if "debug_names" in refs else {},
        io_aliases=_io_aliases(sec("io_aliases")) if "io_aliases" in refs else [],
        input_roles=_input_roles(sec("input_roles")) if "input_roles" in refs else [],
    )
    _validate(pkg)
    return pkg


def _validate(pkg):
    """The cross-checks of parse.zig:161 (`validateGraphMeta`) and the index checks a consumer relies on."""
    gm = pkg.graph_meta
    counts = {"values": len(pkg.values), "nodes": len(pkg.nodes), "regions": len(pkg.regions), "initializers": len(pkg.tensors),
              "inputs": len(pkg.inputs), "outputs": len(pkg.outputs), "dim_symbols": len(pkg.dim_symbols),
              "dim_exprs": len(pkg.dim_exprs), "metadata": len(pkg.metadata), "debug_names": len(pkg.debug_names),
              "io_aliases": len(pkg.io_aliases)}
    for k, n in counts.items():
        if gm[k] != n:
            raise PackageError("InvalidFormat", "graph_meta says %d %s, the sections hold %d" % (gm[k], k, n))
    nv = len(pkg.values)
    for v in pkg.values:
        if v.rank != len(v.shape) or (v.initializer is not None and v.initializer >= len(pkg.tensors)):
            raise PackageError("InvalidFormat", "value record")
        for kind, payload in v.shape:
            if kind == "expr" and payload >= len(pkg.dim_exprs):
                raise PackageError("InvalidFormat", "dimension expression index")
    for n in pkg.nodes:
        if n.output >= nv or any(i >= nv for i in n.inputs) or any(i >= nv for i in n.extra_outputs):
            raise PackageError("InvalidFormat", "node refers to value outside the table")
    for _name, vid in pkg.inputs + pkg.outputs:
        if vid >= nv:
            raise PackageError("InvalidFormat", "signature refers to value outside the table")


def load(path):
    """Maps the file read-only and parses it; tensor payloads stay views of the mapping."""
    with open(path, "rb") as fh:
        mapping = mmap.mmap(fh.fileno(), 0, access=mmap.ACCESS_READ)
    pkg = parse(mapping)
    pkg._mapping = mapping
    return pkg
