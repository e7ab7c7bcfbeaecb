"""A Session over a step list (backend/backend.zig:24-52 Session.execute) on the native executor.

`Steps` writes the records an aion binding would make from an ExecutableProgram's `steps`
(runtime/executable.zig:302-345): one record per step, every TensorId replaced by what the tensor
store answers for it (device address, dtype, shape). Field names follow the Step structs
(StepMatMul a/b/c/alpha/beta, StepRMSNorm x/gamma/beta/residual/eps, ...). `Session.execute`
hands the array to `aionhip_session_execute`; tag dispatch, shape arithmetic, the re-laid weight
cache and the step patterns run in the library.
"""
import ctypes as C

import numpy as np

from . import hip
from .hip import F16, F32, I32, Step, TensorRef

# Step union tags in declaration order (runtime/executable.zig:302-345)
MATMUL, ELEMWISE_BINARY, UNARY, RMSNORM, ATTENTION, ARGMAX, COPY, GATHER_ROWS, GATHER = 0, 1, 2, 8, 9, 11, 17, 18, 19
ROPE1D, SEQUENCE_APPEND, CAST, MATMUL_NT, TRANSFER = 21, 22, 31, 32, 33
# ElemwiseBinaryOp / UnaryOp / ElementwiseBroadcastKind ids (backend/types.zig:92-128, runtime/executable.zig:28-35)
ADD, SUB, MUL, DIV, GATE = 0, 1, 2, 3, 10
RELU, GELU, SILU, SIGMOID, TANH, SQRT, LOG = range(7)
IDENTICAL, SCALAR_A, SCALAR_B, SUFFIX_A, SUFFIX_B, GENERIC = range(6)
ROLLING, WORKSPACE = 1, 2
FUSE_SIBLINGS, FUSE_WORKSPACE = 1, 2


def tensor(buf, dtype, shape, rolling=False, workspace=False, offset=0):
    """A TensorRef for the device buffer `buf` (None: the step has no such operand)."""
    t = TensorRef()
    if buf is None:
        return t
    t.handle = buf.handle + offset
    t.dtype = dtype
    t.rank = len(shape)
    t.flags = (ROLLING if rolling else 0) | (WORKSPACE if workspace else 0)
    for i, d in enumerate(shape):
        t.shape[i] = d
    return t


class Steps:
    """The step records of one program, in order."""

    def __init__(self):
        self.records = []
        self._keep = []

    def _add(self, tag, out, ins, **attrs):
        s = Step()
        s.tag = tag
        if out is not None:
            s.out = out
        for i, t in enumerate(ins):
            if t is not None:
                s.in_[i] = t
        for k, v in attrs.items():
            setattr(s, k, v)
        self.records.append(s)
        return s

    def matmul(self, a, b, c, alpha=1.0, beta=0.0):
        return self._add(MATMUL, c, [a, b], alpha=alpha, beta=beta)

    def matmul_nt(self, a, b, c, alpha=1.0, beta=0.0):
        return self._add(MATMUL_NT, c, [a, b], alpha=alpha, beta=beta)

    def elemwise_binary(self, op, a, b, out, broadcast=IDENTICAL, act=RELU):
        return self._add(ELEMWISE_BINARY, out, [a, b], op=op, broadcast=broadcast, act=act)

    def unary(self, op, a, out):
        return self._add(UNARY, out, [a], op=op)

    def rmsnorm(self, x, gamma, beta, out, eps, residual=None):
        return self._add(RMSNORM, out, [x, gamma, beta, residual], eps=eps)

    def attention(self, q, k, v, out, scale, window=(hip.UNBOUNDED, 0, 0), soft_cap=0.0, query_positions=None, kv_lengths=None):
        return self._add(ATTENTION, out, [q, k, v, query_positions, kv_lengths], scale=scale, soft_cap=soft_cap,
                         window_left=window[0], window_right=window[1], window_chunk=window[2])

    def argmax(self, a, out, axis):
        return self._add(ARGMAX, out, [a], axis=axis)

    def copy(self, src, dst):
        return self._add(COPY, dst, [src])

    def gather_rows(self, table, indices, out):
        return self._add(GATHER_ROWS, out, [table, indices])

    def gather(self, data, indices, out, axis=0, batch_dims=0):
        return self._add(GATHER, out, [data, indices], axis=axis, batch_dims=batch_dims)

    def rope1d(self, x, positions, out, base_frequency=10000.0, scale_factor=1.0, rope_proportion=1.0):
        return self._add(ROPE1D, out, [x, positions], rope_base=base_frequency, rope_scale=scale_factor, rope_proportion=rope_proportion)

    def sequence_append(self, cache, new_kv, end_index):
        return self._add(SEQUENCE_APPEND, cache, [new_kv, end_index])

    def cast(self, x, out):
        return self._add(CAST, out, [x])

    def transfer_to_host(self, src, host_array):
        """Device tensor -> the bytes of `host_array` (a writable C-contiguous numpy array of the tensor's size)."""
        assert host_array.flags.c_contiguous and host_array.flags.writeable
        self._keep.append(host_array)
        return self._add(TRANSFER, None, [src], to_host=1, host=host_array.ctypes.data, host_bytes=host_array.nbytes)

    def transfer_to_device(self, host_array, dst):
        host_array = np.ascontiguousarray(host_array)
        self._keep.append(host_array)
        return self._add(TRANSFER, dst, [], to_host=0, host=host_array.ctypes.data, host_bytes=host_array.nbytes)

    def raw(self, tag, out=None, ins=(), **attrs):
        """A record with any tag (the executor answers Unsupported for the ones it does not run)."""
        return self._add(tag, out, list(ins), **attrs)

    def array(self):
        arr = (Step * len(self.records))()
        for i, s in enumerate(self.records):
            C.memmove(C.byref(arr, i * C.sizeof(Step)), C.byref(s), C.sizeof(Step))
        return arr


class Session:
    """Backend.createSession: executes step lists on one HipBackend's context and keeps the re-laid weights."""

    def __init__(self, backend):
        self._be = backend
        self._lib = backend._lib
        p = C.c_void_p()
        backend._check(self._lib.aionhip_session_create(backend._ctx, C.byref(p)))
        self._s = p

    def set_fusion(self, mask):
        self._be._check(self._lib.aionhip_session_set_fusion(self._s, mask))

    def execute(self, steps):
        arr = steps.array() if isinstance(steps, Steps) else steps
        self._be._check(self._lib.aionhip_session_execute(self._s, arr, len(arr)))

    def stats(self):
        """-> (calls of the last execute, re-laid weights held, their device bytes)"""
        c, w, b = C.c_uint64(), C.c_uint64(), C.c_uint64()
        self._be._check(self._lib.aionhip_session_stats(self._s, C.byref(c), C.byref(w), C.byref(b)))
        return int(c.value), int(w.value), int(b.value)

    def retire_resources(self):
        self._be._check(self._lib.aionhip_session_retire(self._s))

    def close(self):
        if self._s:
            self._lib.aionhip_session_destroy(self._s)
            self._s = None


__all__ = ["Session", "Steps", "tensor", "F16", "F32", "I32"]
