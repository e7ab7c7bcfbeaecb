"""`.aion` v16 reader (aion_amd/aion_file.py) against packages made by the writer in oracle/aion_writer.py.

What is pinned by a statement other than this repository's own: the header, the section directory, the strings
section and the metadata section are laid out a second time in the reference's Python example
(bindings/python/examples/_common.py:14-57: 72-byte header with magic, u32 version, u32 section count at 8, u64
directory offset at 16; 24-byte entries u32 type, u32 flags, u64 offset, u64 size; strings = u32 count +
length-prefixed strings (type 1); metadata = u32 count + (key, value) string index pairs (type 9)) -
`metadata_by_the_example_layout` below walks a file exactly that way. Tensor, value and node records have no
fixture in the reference: for those the tests are writer -> reader round trips (parity unpinned).
"""
import struct

import numpy as np
import pytest

from aion_amd import aion_file
from oracle import aion_writer

CFG = dict(layers=2, hidden=64, heads=2, kv_heads=1, head_dim=32, ffn=96, vocab=50, eps=1e-6, rope_base=10000.0, wdtype="q4_0")


def fake_blocks(cfg):
    rng = np.random.default_rng(1)
    bb = 18 if cfg["wdtype"] == "q4_0" else 34
    shapes = {"wq": (cfg["hidden"], cfg["heads"] * cfg["head_dim"]), "wk": (cfg["hidden"], cfg["kv_heads"] * cfg["head_dim"]),
              "wv": (cfg["hidden"], cfg["kv_heads"] * cfg["head_dim"]), "wo": (cfg["heads"] * cfg["head_dim"], cfg["hidden"]),
              "wgate": (cfg["hidden"], cfg["ffn"]), "wup": (cfg["hidden"], cfg["ffn"]), "wdown": (cfg["ffn"], cfg["hidden"]),
              "lm_head": (cfg["hidden"], cfg["vocab"])}

    def blocks_of(name):
        k, n = shapes[name.split(".")[-1]]
        return rng.integers(0, 256, (k // 32) * n * bb, dtype=np.uint8)
    return blocks_of


def make(cfg=CFG):
    embed = np.random.default_rng(2).standard_normal((cfg["vocab"], cfg["hidden"])).astype(np.float32)
    return aion_writer.build_decoder_package(cfg, fake_blocks(cfg), embed), embed


def metadata_by_the_example_layout(data):
    """The walk of bindings/python/examples/_common.py:27-57, on bytes instead of a file handle."""
    assert data[:4] == b"AION" and len(data) >= 72
    section_count = struct.unpack_from("<I", data, 8)[0]
    dir_offset = struct.unpack_from("<Q", data, 16)[0]
    sections = {}
    for i in range(section_count):
        stype, _flags, off, size = struct.unpack_from("<IIQQ", data, dir_offset + i * 24)
        sections[stype] = (off, size)
    sb = data[sections[1][0]:sections[1][0] + sections[1][1]]
    n_str = struct.unpack_from("<I", sb, 0)[0]
    pos, strings = 4, []
    for _ in range(n_str):
        ln = struct.unpack_from("<I", sb, pos)[0]
        pos += 4
        strings.append(sb[pos:pos + ln].decode())
        pos += ln
    mb = data[sections[9][0]:sections[9][0] + sections[9][1]]
    n_md = struct.unpack_from("<I", mb, 0)[0]
    return {strings[struct.unpack_from("<I", mb, 4 + i * 8)[0]]: strings[struct.unpack_from("<I", mb, 8 + i * 8)[0]] for i in range(n_md)}, strings


def test_header_directory_strings_metadata_match_the_reference_examples_layout():
    data, _ = make()
    pkg = aion_file.parse(data)
    md, strings = metadata_by_the_example_layout(data)
    assert md == pkg.metadata == {"arch": "synthetic-decoder", "layers": "2"}
    assert strings == pkg.strings
    assert struct.unpack_from("<I", data, 4)[0] == 16                      # version (types.zig:22)
    assert struct.unpack_from("<Q", data, 24)[0] == len(data)              # file size (parse.zig:69)


def test_round_trip_of_a_decoder_package():
    data, embed = make()
    pkg = aion_file.parse(data)
    gm = pkg.graph_meta
    assert gm["values"] == len(pkg.values) and gm["nodes"] == len(pkg.nodes) and gm["initializers"] == len(pkg.tensors)
    assert pkg.dim_symbols == ["seq", "ctx"]
    # inputs with their roles
    assert [n for n, _ in pkg.inputs][:4] == ["tokens", "positions", "write_index", "visible_end"]
    kinds = [pkg.role_of_input(i).kind for i in range(len(pkg.inputs))]
    assert kinds == ["tokens", "positions", "cache_write_index", "cache_visible_end"] + ["sequence_cache"] * 4
    assert pkg.role_of_input(4).capacity_symbol == 1 and pkg.role_of_input(4).axis == 1
    # every cache output aliases its cache input
    assert sorted(pkg.io_aliases) == [(4, 2), (5, 3), (6, 4), (7, 5)]
    assert [n for n, _ in pkg.outputs][:2] == ["next_token", "logits"]
    # the node sequence of one layer, as authored
    ops = [n.op for n in pkg.nodes]
    assert ops[0] == "Gather" and ops[-1] == "ArgMax"
    per_layer = ["RMSNorm", "MatMul", "ViewReshape", "MatMul", "ViewReshape", "MatMul", "ViewReshape", "RoPE1D", "RoPE1D", "Cast",
                 "SequenceAppend", "Cast", "SequenceAppend", "Attention", "ViewReshape", "MatMul", "ElemwiseBinary", "RMSNorm",
                 "MatMul", "MatMul", "Unary", "ElemwiseBinary", "MatMul", "ElemwiseBinary"]
    assert ops[1:1 + len(per_layer)] == per_layer
    att = next(n for n in pkg.nodes if n.op == "Attention")
    assert att.attrs["window"] == {"left": 0xFFFFFFFF, "right": 0, "chunk": 0} and att.attrs["has_query_positions"] and att.attrs["has_kv_lengths"]
    assert abs(att.attrs["scale"] - 1 / np.sqrt(32)) < 1e-7 and len(att.inputs) == 5
    rope = next(n for n in pkg.nodes if n.op == "RoPE1D")
    assert rope.attrs == {"base_frequency": 10000.0, "scale_factor": 1.0, "rope_proportion": 1.0}
    # symbolic shapes
    logits_vid = dict(pkg.outputs)["logits"]
    assert pkg.shape_of(logits_vid, {"seq": 7, "ctx": 16}) == (1, 7, 50)
    assert pkg.shape_of(pkg.inputs[4][1], {"seq": 7, "ctx": 16}) == (1, 16, 1, 32)
    with pytest.raises(aion_file.PackageError):
        pkg.shape_of(logits_vid, {})
    # tensors: payloads are views at 64-byte file offsets, bytes intact
    base = np.frombuffer(data, np.uint8).ctypes.data
    for t in pkg.tensors:
        assert (t.data.ctypes.data - base) % 64 == 0
    table = pkg.tensors[pkg.values[pkg.nodes[0].inputs[0]].initializer]
    assert not table.quantized and table.dtype == "f32"
    assert np.array_equal(np.frombuffer(table.data, np.float32).reshape(embed.shape), embed)
    wq = next(t for t in pkg.tensors if t.quantized)
    assert wq.scheme == "q4_0" and wq.block_elems == 32 and wq.block_bytes == 18 and wq.quant_axis == 0
    assert wq.data.size == (64 // 32) * 64 * 18


def test_q8_weights_are_stored_rows_major_under_a_transpose_view():
    data, _ = make(dict(CFG, wdtype="q8_0"))
    pkg = aion_file.parse(data)
    mm = next(n for n in pkg.nodes if n.op == "MatMul")
    tr = next(n for n in pkg.nodes if n.output == mm.inputs[1])
    assert tr.op == "ViewTranspose2D"
    w = pkg.values[tr.inputs[0]]
    t = pkg.tensors[w.initializer]
    assert w.dtype == "q8_0" and t.scheme == "q8_0" and t.quant_axis == 1 and t.block_bytes == 34
    assert pkg.shape_of(tr.inputs[0], {}) == (64, 64) and pkg.shape_of(tr.output, {}) == (64, 64)


def test_malformed_files_are_refused():
    data, _ = make()
    pe = aion_file.PackageError
    with pytest.raises(pe, match="InvalidFormat"):
        aion_file.parse(b"NOPE" + data[4:])
    with pytest.raises(pe, match="UnsupportedVersion"):
        aion_file.parse(data[:4] + struct.pack("<I", 15) + data[8:])
    with pytest.raises(pe, match="InvalidFormat"):
        aion_file.parse(data[:-1])                                         # file size field no longer matches
    with pytest.raises(pe, match="InvalidFormat"):
        aion_file.parse(data[:40])
    # an unknown section type: skipped when optional, refused when required (parse.zig:185-188)
    n = struct.unpack_from("<I", data, 8)[0]
    last = 72 + (n - 1) * 24
    optional = bytearray(data)
    struct.pack_into("<I", optional, last, 99)
    assert aion_file.parse(bytes(optional)).input_roles == []             # the last section was input_roles
    required = bytearray(optional)
    struct.pack_into("<I", required, last + 4, 1)
    with pytest.raises(pe, match="UnsupportedFeature"):
        aion_file.parse(bytes(required))
    # a required section that is not flagged required (parse.zig:193-195)
    unflagged = bytearray(data)
    struct.pack_into("<I", unflagged, 72 + 4, 0)
    with pytest.raises(pe, match="InvalidFormat"):
        aion_file.parse(bytes(unflagged))
    # graph_meta that disagrees with the sections
    idx = [struct.unpack_from("<I", data, 72 + i * 24)[0] for i in range(n)].index(6)
    off = struct.unpack_from("<Q", data, 72 + idx * 24 + 8)[0]
    wrong = bytearray(data)
    struct.pack_into("<I", wrong, off + 4, 1)                              # node count
    with pytest.raises(pe, match="InvalidFormat"):
        aion_file.parse(bytes(wrong))


def test_load_maps_the_file(tmp_path):
    data, embed = make()
    path = tmp_path / "tiny.aion"
    path.write_bytes(data)
    pkg = aion_file.load(str(path))
    table = pkg.tensors[pkg.values[pkg.nodes[0].inputs[0]].initializer]
    assert not table.data.flags.writeable
    assert np.array_equal(np.frombuffer(table.data, np.float32).reshape(embed.shape), embed)


def test_byte_mutations_raise_only_package_errors():
    # every mutated file either parses or is refused with PackageError - never another exception type (the string table is
    # raw bytes in aion, parse.zig:272-284: bytes that are not UTF-8 must not fail the reader)
    data, _ = make()
    rng = np.random.default_rng(123)
    # the structured part of the file: header, directory and every section but the bulk tensor payloads
    n = struct.unpack_from("<I", data, 8)[0]
    spans = [(0, 72 + n * 24)]
    for i in range(n):
        stype, _f, off, size = struct.unpack_from("<IIQQ", data, 72 + i * 24)
        spans.append((off, min(size, 4096) if stype == 2 else size))
    positions = np.concatenate([np.arange(o, o + s) for o, s in spans])
    outcomes = {"ok": 0, "refused": 0}
    for _ in range(3000):
        m = bytearray(data)
        for _k in range(int(rng.integers(1, 4))):
            m[int(rng.choice(positions))] = int(rng.integers(0, 256))
        try:
            aion_file.parse(bytes(m))
            outcomes["ok"] += 1
        except aion_file.PackageError:
            outcomes["refused"] += 1
    assert outcomes["refused"] > 100 and outcomes["ok"] > 100, outcomes
    # a string that is not UTF-8 survives as its bytes
    sidx = [struct.unpack_from("<I", data, 72 + i * 24)[0] for i in range(n)].index(1)
    soff = struct.unpack_from("<Q", data, 72 + sidx * 24 + 8)[0]
    first_len = struct.unpack_from("<I", data, soff + 4)[0]
    assert first_len > 0
    m = bytearray(data)
    m[soff + 8] = 0xFF
    pkg = aion_file.parse(bytes(m))
    assert pkg.strings[0].encode("utf-8", "surrogateescape") == bytes(m[soff + 8:soff + 8 + first_len])
