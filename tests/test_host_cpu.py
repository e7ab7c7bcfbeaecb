"""CPU-side checks of the product library: the host quantizer is byte-exact against the oracle,
the shared library loads and exports every entry point the header declares."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from aion_amd import backend as be
from aion_amd import hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    lib = hip.load_library()
    text = open(os.path.join(ROOT, "include", "aion_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = set(re.findall(r"\b(aionhip_[a-z0-9_]+)\s*\(", text))
    assert len(names) >= 35
    missing = [n for n in sorted(names) if not hasattr(lib, n)]
    assert not missing, missing
    untyped = [n for n in sorted(names) if n not in hip._SIGS]
    assert not untyped, untyped


@pytest.mark.parametrize("dtype", [be.Q8_0, be.Q4_0])
@pytest.mark.parametrize("shape,axis", [((64, 5), 0), ((7, 96), 1), ((2, 64, 3), 1), ((4096, 24), 0), ((300, 512), 1)])
def test_host_quantizer_matches_oracle_bytes(orc, dtype, shape, axis):
    rng = np.random.default_rng(hash((dtype, shape, axis)) % 2**32)
    v = (rng.standard_normal(shape) * 0.02).astype(np.float32)
    v.reshape(-1)[::97] = 0.0
    if v.ndim == 2 and axis == 1:
        v[0, :32] = 0.0                       # an all-zero block
    got = be.quantize_blocks(dtype, v, axis)
    want = orc.quantize(dtype, v, axis)
    assert np.array_equal(got, want)


def test_host_quantizer_reference_test_vector(orc):
    # aion storage/quantize.zig:105-137
    i = np.arange(64 * 5)
    vals = ((i % 17).astype(np.int32) - 8).astype(np.float32) * np.float32(0.1)
    got = be.quantize_blocks(be.Q8_0, vals.reshape(64, 5), 0)
    assert np.array_equal(got, orc.quantize(orc.Q8_0, vals.reshape(64, 5), 0))


def test_host_q4_quantizer_divides_by_the_unrounded_scale():
    # the hand-computed block of test_oracle_quant.py (max_abs = 7 * (1 + 2^-12): stored scale f16 1.0, codes from the f32 scale)
    v = np.zeros((1, 32), np.float32)
    v[0, :4] = [7.0 + 7.0 / 4096.0, 2.5, -2.5, 0.5]
    want = bytes([0x00, 0x3C, 15 | (10 << 4), 6 | (8 << 4)] + [0x88] * 14)
    assert be.quantize_blocks(be.Q4_0, v, 1).tobytes() == want
    assert be.quantize_blocks(be.Q4_0, np.ascontiguousarray(v.T), 0).tobytes() == want


def test_host_quantizer_chunked_calls_equal_whole():
    # api/context.zig:443-489 quantizes 16 MiB at a time through first_elem/first_block
    lib = hip.load_library()
    rng = np.random.default_rng(3)
    v = rng.standard_normal((8, 128)).astype(np.float32)
    whole = be.quantize_blocks(be.Q8_0, v, 1)
    shape = (C.c_size_t * 2)(8, 128)
    parts = []
    for r0 in range(0, 8, 2):
        chunk = np.ascontiguousarray(v[r0:r0 + 2])
        out = np.empty(2 * 4 * 34, np.uint8)
        rc = lib.aionhip_quantize_blocks(be.Q8_0, shape, 2, 1, chunk.ctypes.data, chunk.size, r0 * 128, r0 * 4, out.ctypes.data, out.nbytes)
        assert rc == hip.OK
        parts.append(out)
    assert np.array_equal(np.concatenate(parts), whole)


def test_host_quantizer_errors():
    with pytest.raises(be.AionHipError) as e:
        be.quantize_blocks(be.Q8_0, np.zeros((33, 4), np.float32), 0)
    assert e.value.status == hip.INVALID_ARGUMENT
    with pytest.raises(be.AionHipError) as e:
        be.quantize_blocks(be.F16, np.zeros((32, 4), np.float32), 0)
    assert e.value.status == hip.UNSUPPORTED
    lib = hip.load_library()
    shape = (C.c_size_t * 1)(64)
    v = np.zeros(32, np.float32)      # too few values for two blocks
    out = np.empty(68, np.uint8)
    assert lib.aionhip_quantize_blocks(be.Q8_0, shape, 1, 0, v.ctypes.data, v.size, 0, 0, out.ctypes.data, 68) == hip.INVALID_ARGUMENT


def test_create_without_gpu_fails_loudly():
    import subprocess
    import sys
    # in a child process so that a GPU-less HIP runtime cannot disturb this one
    code = ("import sys; sys.path.insert(0, %r)\n"
            "from aion_amd import backend as be\n"
            "try:\n    be.HipBackend(7)\n    print('created')\n"
            "except be.AionHipError as e:\n    print('error', e.status)\n") % ROOT
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120).stdout
    assert "error" in out          # device 7 never exists on a one-GPU box or a CPU container


def test_ctypes_structures_have_the_header_layout(tmp_path):
    """The records a binding fills (attention parameters, tensor references, steps) as a C compiler lays them out from
    include/aion_hip.h, field by field, against the ctypes mirrors the harness passes."""
    import subprocess
    mirrors = {"aionhip_attention": hip.Attention, "aionhip_tensor_ref": hip.TensorRef, "aionhip_step": hip.Step}
    lines = []
    for cname, mirror in mirrors.items():
        lines.append('printf("%s size %%zu\\n", sizeof(%s));' % (cname, cname))
        for field, _ in mirror._fields_:
            lines.append('printf("%s %s %%zu\\n", offsetof(%s, %s));' % (cname, field, cname, field.rstrip("_")))
    src = tmp_path / "layout.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "aion_hip.h"\nint main(void) {\n%s\nreturn 0; }\n' % "\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split("\n")
    seen = 0
    for line in filter(None, out):
        cname, field, value = line.split()
        mirror = mirrors[cname]
        if field == "size":
            assert C.sizeof(mirror) == int(value), cname
        else:
            assert getattr(mirror, field).offset == int(value), (cname, field)
        seen += 1
    assert seen == sum(len(m._fields_) + 1 for m in mirrors.values())
    # the step tags are the Step union's tags in declaration order (runtime/executable.zig:302-345)
    from aion_amd import session as ss
    order = ["MatMul", "ElemwiseBinary", "Unary", "Softmax", "Conv1D", "Conv2D", "MaxPool2D", "LayerNorm", "RMSNorm", "Attention", "RelPosMHA",
             "ArgMax", "TopK", "ScatterRow", "ReduceAll", "ReduceAxis", "ConcatScalar", "Copy", "GatherRows", "Gather", "GatherND", "RoPE1D",
             "SequenceAppend", "LSTMCellFused", "If", "Loop", "RFFT", "STFT", "ReshapeScalar", "Transpose2DScalar", "SliceNDScalar", "Cast",
             "MatMulNT", "Transfer"]
    header = open(os.path.join(ROOT, "include", "aion_hip.h")).read()
    for name, const in (("MatMul", "MATMUL"), ("ElemwiseBinary", "ELEMWISE_BINARY"), ("Unary", "UNARY"), ("RMSNorm", "RMSNORM"),
                        ("Attention", "ATTENTION"), ("ArgMax", "ARGMAX"), ("Copy", "COPY"), ("GatherRows", "GATHER_ROWS"), ("Gather", "GATHER"),
                        ("RoPE1D", "ROPE1D"), ("SequenceAppend", "SEQUENCE_APPEND"), ("Cast", "CAST"), ("MatMulNT", "MATMUL_NT"),
                        ("Transfer", "TRANSFER")):
        assert getattr(ss, const) == order.index(name)
        assert re.search(r"AIONHIP_STEP_%s = %d\b" % (const, order.index(name)), header), const
    assert re.search(r"AIONHIP_STEP_TAG_COUNT = %d\b" % len(order), header)


def test_session_entry_points_reject_null_handles_without_a_gpu():
    lib = hip.load_library()
    p = C.c_void_p()
    assert lib.aionhip_session_create(None, C.byref(p)) == hip.INVALID_ARGUMENT
    assert lib.aionhip_session_execute(None, None, 0) == hip.INVALID_ARGUMENT
    assert lib.aionhip_session_set_fusion(None, 3) == hip.INVALID_ARGUMENT
    assert lib.aionhip_session_retire(None) == hip.INVALID_ARGUMENT
    assert lib.aionhip_session_stats(None, None, None, None) == hip.INVALID_ARGUMENT
    lib.aionhip_session_destroy(None)          # a no-op
