"""The `.aion` v16 reader (aion_amd/aion_file.py) against a package assembled HERE byte by byte from the layouts the
reference's parser states - not through oracle/aion_writer.py, so a mistake shared by this repository's writer and
reader (a swapped field, a wrong pad, a wrong enum id) does not cancel out. Every `struct.pack` below cites the lines of
storage/aion_file/parse.zig (or the enum it reads) that fix the layout:

  header 72 B                      parse.zig:59-69      magic, u32 version, u32 sections, u32 0, u64 dir offset, u64 file size, u64 flags, 32 B
  directory entry 24 B             parse.zig:175-196    u32 type, u32 flags (bit 0 = required), u64 offset, u64 size
  strings                          parse.zig:272-284    u32 count, count x (u32 len, bytes)
  dim symbols / expressions        parse.zig:291-327    u32 count x u32 string idx;  u8 kind, 3 B pad, u32 aux, ShapeTerm lhs, rhs
  ShapeTerm 16 B                   parse.zig:827-836    u8 kind (0 constant, 1 expression), 7 B pad, u64 payload
  tensors                          parse.zig:329-381    u8 kind, u8 plain dtype, u8 logical dtype, u8 0, u32 scheme idx, u32 block elems,
                                                        u32 block bytes, i32 quant axis, u32 params len, u64 data len, params, zero pad to a
                                                        multiple of 64 measured from the SECTION start, data
  values                           parse.zig:383-408    u8 dtype, u8 rank, u8 source, u8 0, u32 initializer | ~0, u32 terms, terms
  nodes                            parse.zig:410-439    u16 op, u16 0, u32 output, u32 inputs, u32 attr bytes, inputs, attrs
  node attributes                  parse.zig:485-640    per op (see each node below)
  signatures                       parse.zig:642-671    u32 inputs, u32 outputs, then (u32 name idx, u32 value) each
  graph meta                       parse.zig:750-767    11 x u32
  metadata / debug names / aliases parse.zig:673-720    (u32 key, u32 value) / (u32 value, u32 name) / (u32 input, u32 output)
  input roles                      parse.zig:722-748    u32 input, u8 kind, u8 axis, u8 flags, u8 0, u32 capacity symbol, u32 retained
Enum ids: DType (backend/types.zig:29-38) f32 0, f16 1, i8 2, q4_0 3, q8_0 4, i32 5; OpTag (graph/graph.zig:62-128);
ElemwiseBinaryOp / UnaryOp (backend/types.zig:92-127); ValueSource, InputRoleKind (storage/aion_file/types.zig:127-131, 164-177);
section types (types.zig:40-54).
"""
import struct

import numpy as np
import pytest

from aion_amd import aion_file

INVALID = 0xFFFFFFFF


def term(kind, payload):
    return struct.pack("<B7xQ", kind, payload)


def const(n):
    return term(0, n)


def expr(i):
    return term(1, i)


def sym_attr(*terms):
    return struct.pack("<I", len(terms)) + b"".join(terms)


def node(op, output, inputs, attrs=b""):
    return struct.pack("<HHIII", op, 0, output, len(inputs), len(attrs)) + struct.pack("<%dI" % len(inputs), *inputs) + attrs


def value(dtype, source, shape_terms, initializer=INVALID):
    return struct.pack("<BBBBII", dtype, len(shape_terms), source, 0, initializer, len(shape_terms)) + b"".join(shape_terms)


STRINGS = ["q4_0", "tokens", "cache", "pos", "logits", "next", "seq", "ctx", "arch", "by-hand", "w_head", "q8_0"]
S = {s: i for i, s in enumerate(STRINGS)}

# two quant blocks of a q4_0 [K = 32, N = 2] operand (18 bytes each) and a plain f32 vector
Q4_BLOCKS = bytes(range(1, 37))
F32_DATA = np.arange(5, dtype=np.float32).tobytes()
Q8_PARAMS = b"\x07\x09\x0b"


def tensors_section():
    out = struct.pack("<I", 3)
    # quantized: kind 1, plain dtype ignored (0), logical dtype f32 (0), scheme "q4_0", 32 elements in 18 bytes, quant axis 0
    out += struct.pack("<BBBBIIIiIQ", 1, 0, 0, 0, S["q4_0"], 32, 18, 0, 0, len(Q4_BLOCKS))
    out += b"\0" * (-len(out) % 64) + Q4_BLOCKS
    # plain f32: kind 0, dtype 0, no scheme
    out += struct.pack("<BBBBIIIiIQ", 0, 0, 0, 0, INVALID, 0, 0, 0, 0, len(F32_DATA))
    out += b"\0" * (-len(out) % 64) + F32_DATA
    # quantized with params (3 bytes in front of the pad), logical dtype f16 (1), scheme "q8_0", quant axis -1, no data bytes
    out += struct.pack("<BBBBIIIiIQ", 1, 0, 1, 0, S["q8_0"], 32, 34, -1, len(Q8_PARAMS), 0) + Q8_PARAMS
    out += b"\0" * (-len(out) % 64)
    return out


def build():
    strings = struct.pack("<I", len(STRINGS)) + b"".join(struct.pack("<I", len(s)) + s.encode() for s in STRINGS)
    dim_symbols = struct.pack("<II", 2, S["seq"]) + struct.pack("<I", S["ctx"])
    # expressions: 0 = symbol 0 (seq), 1 = symbol 1 (ctx), 2 = seq * 8, 3 = max(ctx, 4), 4 = (ctx - 1) / 2, 5 = seq + ctx
    dim_exprs = struct.pack("<I", 6) + b"".join([
        struct.pack("<B3xI", 0, 0) + const(0) + const(0),
        struct.pack("<B3xI", 0, 1) + const(0) + const(0),
        struct.pack("<B3xI", 3, 0) + expr(0) + const(8),
        struct.pack("<B3xI", 5, 0) + expr(1) + const(4),
        struct.pack("<B3xI", 4, 0) + expr(5) + const(2),        # floor_div of expression 5 (below: seq + ctx) by 2
        struct.pack("<B3xI", 1, 0) + expr(0) + expr(1),
    ])
    values = struct.pack("<I", 9) + b"".join([
        value(5, 0, [const(1), expr(0)]),                        # 0 tokens   i32 [1, seq]        input
        value(1, 0, [const(1), expr(1), const(1), const(32)]),   # 1 cache    f16 [1, ctx, 1, 32] input
        value(5, 0, [const(1), expr(0)]),                        # 2 pos      i32 [1, seq]        input
        value(3, 1, [const(32), const(2)], initializer=0),       # 3 w        q4_0 [32, 2]        initializer 0
        value(0, 1, [const(5)], initializer=1),                  # 4 gamma    f32 [5]             initializer 1
        value(0, 2, [const(1), expr(0), const(2)]),              # 5 produced f32 [1, seq, 2]
        value(0, 2, [expr(2)]),                                  # 6 produced f32 [seq * 8]
        value(5, 2, [const(1), expr(0)]),                        # 7 produced i32 [1, seq]
        value(1, 2, [const(1), expr(3), const(1), const(32)]),   # 8 produced f16 [1, max(ctx, 4), 1, 32]
    ])
    f32 = lambda x: struct.pack("<f", x)
    nodes = [
        node(0, 5, [0, 3], f32(0.5) + f32(2.0)),                                             # MatMul{alpha, beta}
        node(1, 5, [5, 5], struct.pack("<B", 9)),                                            # ElemwiseBinary{ge = 9}
        node(2, 5, [5], struct.pack("<B", 1)),                                               # Unary{gelu = 1}
        node(7, 5, [5, 4], f32(1e-6) + sym_attr(const(2))),                                  # RMSNorm{eps, normalized shape}
        node(19, 5, [5, 1, 1, 2, 2], f32(0.0625) + struct.pack("<III", 0xFFFFFFFF, 0, 64) + f32(30.0) + struct.pack("<B", 3)),   # Attention
        node(17, 5, [5, 2], f32(10000.0) + f32(1.0) + f32(0.5)),                             # RoPE1D{base, scale, proportion}
        node(20, 8, [5], struct.pack("<B", 1)),                                              # Cast{f16 = 1}
        node(18, 8, [1, 8, 2]),                                                              # SequenceAppend{}
        node(12, 6, [5], sym_attr(expr(2))),                                                 # ViewReshape{[seq * 8]} - a free axis
        node(16, 6, [6], struct.pack("<IQ", 1, 3) + sym_attr(const(4))),                     # ViewSliceND{starts [3], lens [4]}
        node(13, 6, [6], struct.pack("<Bi", 1, -1)),                                         # ViewSqueeze{axis -1}
        node(13, 6, [6], struct.pack("<B", 0)),                                              # ViewSqueeze{no axis}
        node(14, 6, [6], struct.pack("<i", 0)),                                              # ViewUnsqueeze{axis 0}
        node(15, 6, [6]),                                                                    # ViewTranspose2D{}
        node(28, 5, [4, 0], struct.pack("<iQ", 0, 1)),                                       # Gather{axis, batch dims}
        node(26, 7, [5], struct.pack("<i", -1)),                                             # ArgMax{axis}
        node(11, 7, [7]),                                                                    # Copy{}
        node(3, 5, [5], struct.pack("<i", 2)),                                               # Softmax{axis}
        node(8, 5, [5], struct.pack("<BBi", 1, 1, 1)),                                       # Reduce{mean = 1, axis 1}
        node(9, 5, [5, 5], struct.pack("<i", -1)),                                           # Concat{axis}
        node(31, 5, [5], struct.pack("<QiBII", 3, -1, 1, 1, 7)),                             # TopK{k, axis, largest, 1 extra output: value 7}
    ]
    nodes_sec = struct.pack("<I", len(nodes)) + b"".join(nodes)
    signatures = struct.pack("<II", 3, 2) + struct.pack("<II", S["tokens"], 0) + struct.pack("<II", S["cache"], 1) + struct.pack("<II", S["pos"], 2) + \
        struct.pack("<II", S["logits"], 5) + struct.pack("<II", S["next"], 7)
    metadata = struct.pack("<III", 1, S["arch"], S["by-hand"])
    debug_names = struct.pack("<III", 1, 3, S["w_head"])
    io_aliases = struct.pack("<III", 1, 1, 0)
    input_roles = struct.pack("<I", 3) + struct.pack("<IBBBBII", 1, 1, 1, 3, 0, 1, 7) + struct.pack("<IBBBBII", 2, 4, 1, 1, 0, INVALID, 0) + \
        struct.pack("<IBBBBII", 0, 5, 1, 1, 0, INVALID, 0)
    graph_meta = struct.pack("<11I", 9, len(nodes), 0, 3, 3, 2, 2, 6, 1, 1, 1)

    # writer order of the reference (write.zig:49-61) is not required by the reader; here: strings, dim symbols, dim expressions, an
    # unknown optional section, then the tensors on a 64-byte offset, and the rest
    sections = [(1, 1, strings), (7, 0, dim_symbols), (8, 0, dim_exprs), (99, 0, b"ignored"), (2, 1, tensors_section()), (3, 1, values),
                (4, 1, nodes_sec), (5, 1, signatures), (6, 1, graph_meta), (9, 0, metadata), (10, 0, debug_names), (12, 0, io_aliases),
                (13, 0, input_roles)]
    body = b""
    directory = b""
    base = 72 + 24 * len(sections)
    for stype, flags, payload in sections:
        if stype == 2:
            body += b"\0" * (-(base + len(body)) % 64)
        directory += struct.pack("<IIQQ", stype, flags, base + len(body), len(payload))
        body += payload
    total = base + len(body)
    header = b"AION" + struct.pack("<III", 16, len(sections), 0) + struct.pack("<QQQ", 72, total, 0) + b"\0" * 32
    assert len(header) == 72
    return header + directory + body


def test_every_record_type_built_by_hand_parses_to_what_was_written():
    pkg = aion_file.parse(build())
    assert pkg.strings == STRINGS
    assert pkg.dim_symbols == ["seq", "ctx"]
    assert pkg.dim_exprs[2] == ("mul", 0, ("expr", 0), ("const", 8)) and pkg.dim_exprs[3] == ("max", 0, ("expr", 1), ("const", 4))
    assert pkg.dim_exprs[4][0] == "floor_div" and pkg.dim_exprs[5][0] == "add" and pkg.dim_exprs[0][:2] == ("symbol", 0) and pkg.dim_exprs[1][:2] == ("symbol", 1)
    sym = {"seq": 3, "ctx": 10}
    assert pkg.shape_of(5, sym) == (1, 3, 2) and pkg.shape_of(6, sym) == (24,) and pkg.shape_of(8, sym) == (1, 10, 1, 32)
    assert pkg.dim_term(("expr", 4), sym) == (3 + 10) // 2
    # tensors: the payloads sit on 64-byte offsets of the section, behind the params
    q4, plain, q8 = pkg.tensors
    assert q4.quantized and q4.scheme == "q4_0" and q4.dtype == "f32" and (q4.block_elems, q4.block_bytes, q4.quant_axis) == (32, 18, 0)
    assert bytes(q4.data) == Q4_BLOCKS and q4.params == b""
    assert not plain.quantized and plain.dtype == "f32" and np.array_equal(np.frombuffer(bytes(plain.data), np.float32), np.arange(5, dtype=np.float32))
    assert q8.quantized and q8.scheme == "q8_0" and q8.dtype == "f16" and q8.quant_axis == -1 and q8.params == Q8_PARAMS and q8.data.size == 0
    # values
    v = pkg.values
    assert (v[0].dtype, v[0].rank, v[0].source, v[0].initializer) == ("i32", 2, "input", None)
    assert (v[1].dtype, v[1].source, v[1].shape[1]) == ("f16", "input", ("expr", 1))
    assert (v[3].dtype, v[3].source, v[3].initializer, v[3].shape) == ("q4_0", "initializer", 0, (("const", 32), ("const", 2)))
    assert (v[4].initializer, v[5].source, v[7].dtype) == (1, "produced", "i32")
    # nodes and their attributes
    n = pkg.nodes
    assert (n[0].op, n[0].output, n[0].inputs, n[0].attrs) == ("MatMul", 5, (0, 3), {"alpha": 0.5, "beta": 2.0})
    assert (n[1].op, n[1].attrs["op"]) == ("ElemwiseBinary", "ge") and (n[2].op, n[2].attrs["op"]) == ("Unary", "gelu")
    assert n[3].op == "RMSNorm" and n[3].attrs["eps"] == pytest.approx(1e-6, rel=1e-6)
    assert [t for t in n[3].attrs.values() if isinstance(t, tuple)] == [(("const", 2),)]
    a = n[4].attrs
    assert n[4].op == "Attention" and n[4].inputs == (5, 1, 1, 2, 2) and a["scale"] == 0.0625
    assert a["window"] == {"left": 0xFFFFFFFF, "right": 0, "chunk": 64}
    assert [a[k] for k in a if "cap" in k] == [30.0]
    assert [bool(a[k]) for k in a if "position" in k or "length" in k] == [True, True]
    assert n[5].op == "RoPE1D" and sorted(n[5].attrs.values()) == [0.5, 1.0, 10000.0]
    assert (n[6].op, list(n[6].attrs.values())) == ("Cast", ["f16"])
    assert (n[7].op, n[7].inputs, n[7].attrs) == ("SequenceAppend", (1, 8, 2), {})
    assert n[8].op == "ViewReshape" and list(n[8].attrs.values()) == [(("expr", 2),)]
    assert n[9].op == "ViewSliceND" and (3,) in [tuple(x) for x in n[9].attrs.values() if not (x and isinstance(x[0], tuple))]
    assert (("const", 4),) in list(n[9].attrs.values())
    assert (n[10].op, n[10].attrs["axis"]) == ("ViewSqueeze", -1) and (n[11].op, n[11].attrs["axis"]) == ("ViewSqueeze", None)
    assert (n[12].op, n[12].attrs["axis"]) == ("ViewUnsqueeze", 0) and (n[13].op, n[13].attrs) == ("ViewTranspose2D", {})
    assert n[14].op == "Gather" and sorted(n[14].attrs.values()) == [0, 1]
    assert (n[15].op, n[15].attrs["axis"]) == ("ArgMax", -1) and (n[16].op, n[16].attrs) == ("Copy", {})
    assert (n[17].op, n[17].attrs["axis"]) == ("Softmax", 2)
    assert n[18].op == "Reduce" and n[18].attrs["op"] == "mean" and n[18].attrs["axis"] == 1
    assert (n[19].op, n[19].attrs["axis"]) == ("Concat", -1)
    assert n[20].op == "TopK" and n[20].extra_outputs == (7,) and n[20].attrs["k"] == 3 and n[20].attrs["axis"] == -1 and bool(n[20].attrs["largest"])
    # signatures, roles, the rest
    assert pkg.inputs == [("tokens", 0), ("cache", 1), ("pos", 2)] and pkg.outputs == [("logits", 5), ("next", 7)]
    assert pkg.metadata == {"arch": "by-hand"} and pkg.debug_names == {3: "w_head"} and pkg.io_aliases == [(1, 0)]
    r = pkg.role_of_input(1)
    assert (r.kind, r.axis, r.flags, r.capacity_symbol, r.retained_history_tokens) == ("sequence_cache", 1, 3, 1, 7)
    assert pkg.role_of_input(2).kind == "positions" and pkg.role_of_input(0).kind == "tokens" and pkg.role_of_input(0).capacity_symbol == INVALID
    assert pkg.graph_meta["values"] == 9 and pkg.graph_meta["initializers"] == 3 and pkg.graph_meta["dim_exprs"] == 6


def test_what_the_reference_parser_rejects_is_rejected():
    good = build()

    def expect(data, kind):
        with pytest.raises(aion_file.PackageError) as e:
            aion_file.parse(data)
        assert e.value.kind == kind, (e.value.kind, kind)

    expect(good[:-1], "InvalidFormat")                                             # file size field != length (parse.zig:69)
    expect(b"AIOM" + good[4:], "InvalidFormat")                                    # magic (parse.zig:165-170)
    expect(good[:4] + struct.pack("<I", 15) + good[8:], "UnsupportedVersion")      # version (parse.zig:168-173)
    # an unknown section type marked required (parse.zig:185-188): entry 3 of the directory is type 99, flags 0 -> set bit 0
    off = 72 + 3 * 24
    assert struct.unpack_from("<I", good, off)[0] == 99
    expect(good[:off + 4] + struct.pack("<I", 1) + good[off + 8:], "UnsupportedFeature")
    # a required section without its required flag (parse.zig:193-196): strings is entry 0
    expect(good[:72 + 4] + struct.pack("<I", 0) + good[72 + 8:], "InvalidFormat")
    # a node whose reserved u16 is not zero (parse.zig:421)
    noff, nsize = [struct.unpack_from("<QQ", good, 72 + i * 24 + 8) for i in range(13) if struct.unpack_from("<I", good, 72 + i * 24)[0] == 4][0]
    bad = bytearray(good)
    bad[noff + 4 + 2] = 1
    expect(bytes(bad), "InvalidFormat")
    # attribute bytes that are not consumed exactly (parse.zig:638): MatMul with 9 attribute bytes instead of 8
    bad = bytearray(good)
    struct.pack_into("<I", bad, noff + 4 + 12, 9)
    with pytest.raises(aion_file.PackageError):
        aion_file.parse(bytes(bad))
