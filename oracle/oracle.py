"""ctypes front end of the CPU oracle (TEST INFRASTRUCTURE ONLY).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
module. It loads oracle/libaion_oracle.so (built by oracle/Makefile) and wraps each
function with numpy in/out. See aion_oracle.h for what each function restates.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libaion_oracle.so")

Q4_0, Q8_0 = 3, 4
BLOCK_BYTES = {Q4_0: 18, Q8_0: 34}
UNBOUNDED = 0xFFFFFFFF


def build():
    subprocess.check_call(["make", "-C", _HERE, "-B", "libaion_oracle.so"], stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = C.CDLL(_LIB_PATH)
    sz, f, i, vp = C.c_size_t, C.c_float, C.c_int, C.c_void_p
    lib.orc_f32_to_f16.argtypes = [f]; lib.orc_f32_to_f16.restype = C.c_uint16
    lib.orc_f16_to_f32.argtypes = [C.c_uint16]; lib.orc_f16_to_f32.restype = f
    lib.orc_exp_approx.argtypes = [f]; lib.orc_exp_approx.restype = f
    lib.orc_tanh_approx.argtypes = [f]; lib.orc_tanh_approx.restype = f
    lib.orc_quantize.argtypes = [i, vp, sz, sz, vp, vp]
    lib.orc_dequantize.argtypes = [i, vp, sz, sz, vp, vp]
    lib.orc_prepare_a.argtypes = [vp, sz, sz, sz, vp, vp, vp]; lib.orc_prepare_a.restype = None
    lib.orc_matmul_nt_q8.argtypes = [sz, sz, sz, f, f, vp, sz, vp, vp, sz, i]
    lib.orc_matmul_q8_kmajor.argtypes = [sz, sz, sz, f, f, vp, sz, vp, sz, vp, sz, i]
    lib.orc_matmul_q_packed.argtypes = [i, sz, sz, sz, f, f, vp, sz, vp, vp, sz, sz, i]
    lib.orc_matmul_q_f32a.argtypes = [i, i, sz, sz, sz, f, f, vp, sz, vp, vp, sz, i]
    lib.orc_attention_blocked.argtypes = [vp, vp, vp, vp, vp, vp, vp, i]
    lib.orc_attention_f64.argtypes = [vp, vp, vp, vp, vp, vp, vp]
    lib.orc_rmsnorm.argtypes = [vp, vp, vp, vp, sz, sz, f, vp]; lib.orc_rmsnorm.restype = None
    lib.orc_rope.argtypes = [vp, vp, sz, sz, sz, sz, f, f, f, vp]; lib.orc_rope.restype = None
    lib.orc_gate_gelu.argtypes = [vp, vp, sz, vp]; lib.orc_gate_gelu.restype = None
    lib.orc_unary.argtypes = [C.c_int, vp, sz, vp]; lib.orc_unary.restype = C.c_int
    lib.orc_binary.argtypes = [C.c_int, vp, vp, sz, sz, vp]; lib.orc_binary.restype = C.c_int
    lib.orc_gather_rows.argtypes = [i, vp, sz, vp, sz, vp]; lib.orc_gather_rows.restype = None
    lib.orc_argmax.argtypes = [vp, sz, sz, vp]; lib.orc_argmax.restype = None
    lib.orc_cast_f32_f16.argtypes = [vp, sz, vp]; lib.orc_cast_f32_f16.restype = None
    lib.orc_decoder_create.argtypes = [vp, i]; lib.orc_decoder_create.restype = vp
    lib.orc_decoder_destroy.argtypes = [vp]; lib.orc_decoder_destroy.restype = None
    lib.orc_decoder_set_weight.argtypes = [vp, C.c_char_p, vp, sz]
    lib.orc_decoder_reset.argtypes = [vp]; lib.orc_decoder_reset.restype = None
    lib.orc_decoder_forward.argtypes = [vp, vp, sz, sz, vp]; lib.orc_decoder_forward.restype = C.c_int32
    return lib


_lib = _load()


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def f32_to_f16_bits(v):
    return int(_lib.orc_f32_to_f16(float(np.float32(v))))


def f16_bits_to_f32(b):
    return float(_lib.orc_f16_to_f32(int(b)))


def exp_approx(x):
    return float(_lib.orc_exp_approx(float(np.float32(x))))


def tanh_approx(x):
    return float(_lib.orc_tanh_approx(float(np.float32(x))))


def quantize(dtype, values, quant_axis):
    """f32 array -> packed blocks (uint8), row-major over block space."""
    v = _f32(values)
    shape = (C.c_size_t * v.ndim)(*v.shape)
    out = np.zeros(v.size // 32 * BLOCK_BYTES[dtype], dtype=np.uint8)
    rc = _lib.orc_quantize(dtype, shape, v.ndim, quant_axis, _p(v), _p(out))
    if rc != 0:
        raise ValueError("orc_quantize: InvalidArgument")
    return out


def dequantize(dtype, blocks, shape, quant_axis):
    out = np.zeros(shape, dtype=np.float32)
    sh = (C.c_size_t * len(shape))(*shape)
    b = np.ascontiguousarray(blocks, dtype=np.uint8)
    rc = _lib.orc_dequantize(dtype, sh, len(shape), quant_axis, _p(b), _p(out))
    if rc != 0:
        raise ValueError("orc_dequantize: InvalidArgument")
    return out


def prepare_a(a):
    a = _f32(a)
    m, k = a.shape
    aq = np.zeros((m, k), dtype=np.int8)
    sc = np.zeros((m, k // 32), dtype=np.float32)
    sm = np.zeros((m, k // 32), dtype=np.int32)
    _lib.orc_prepare_a(_p(a), m, k, k, _p(aq), _p(sc), _p(sm))
    return aq, sc, sm


def _c_init(m, n, c, beta):
    if c is None:
        if beta != 0.0:
            raise ValueError("beta != 0 needs c")
        return np.zeros((m, n), dtype=np.float32)
    return np.array(c, dtype=np.float32, copy=True).reshape(m, n)


def matmul_nt_q8(a, b_blocks, n, alpha=1.0, beta=0.0, c=None, threads=1):
    a = _f32(a); m, k = a.shape
    b = np.ascontiguousarray(b_blocks, dtype=np.uint8)
    out = _c_init(m, n, c, beta)
    rc = _lib.orc_matmul_nt_q8(m, n, k, alpha, beta, _p(a), k, _p(b), _p(out), n, threads)
    if rc != 0:
        raise ValueError("orc_matmul_nt_q8: InvalidArgument")
    return out


def matmul_nt_f32(a, b, alpha=1.0, beta=0.0, c=None, lanes=8):
    """MatMulNT with an f32 B [N,K] (cpu/kernels/matmul_nt.zig:40-126): C = alpha * A @ B^T + beta * C. The reference's order:
    four vectors of `lanes` accumulators take k in turns (fused multiply-adds), each is reduced, the four sums are added, the
    K tail past a multiple of 4 * lanes follows element by element; beta == 0 stores alpha * acc. numpy restatement: the
    fused multiply-add is formed in float64 (the product of two f32 is exact there) and rounded to f32, the vector reduce is a
    pairwise tree. Pinned by tests/test_oracle_matmul.py against the float64 product (error bound from K) and on inputs whose
    every partial sum is exact in f32 (small integers), where any summation order gives the same bits."""
    a, b = _f32(a), _f32(b)
    m, k = a.shape
    n = b.shape[0]
    out = _c_init(m, n, c, beta)
    step = 4 * lanes
    k_vec = k - k % step
    acc = np.zeros((m, n, 4, lanes), np.float32)
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    for kk in range(0, k_vec, step):
        pa = a64[:, None, kk:kk + step].reshape(m, 1, 4, lanes)
        pb = b64[None, :, kk:kk + step].reshape(1, n, 4, lanes)
        acc = (pa * pb + acc.astype(np.float64)).astype(np.float32)
    red = acc
    while red.shape[-1] > 1:                                   # @reduce(.Add, v): pairwise
        red = (red[..., 0::2] + red[..., 1::2]).astype(np.float32)
    red = red[..., 0]
    tot = ((red[..., 0] + red[..., 1]).astype(np.float32) + red[..., 2]).astype(np.float32)
    tot = (tot + red[..., 3]).astype(np.float32)
    for kk in range(k_vec, k):
        tot = (tot + (a[:, None, kk] * b[None, :, kk]).astype(np.float32)).astype(np.float32)
    al, be_ = np.float32(alpha), np.float32(beta)
    res = (al * tot).astype(np.float32)
    if beta != 0.0:
        res = (res + (be_ * out).astype(np.float32)).astype(np.float32)
    return res


def matmul_q8_kmajor(a, b_blocks, n, alpha=1.0, beta=0.0, c=None, threads=1):
    a = _f32(a); m, k = a.shape
    b = np.ascontiguousarray(b_blocks, dtype=np.uint8)
    out = _c_init(m, n, c, beta)
    rc = _lib.orc_matmul_q8_kmajor(m, n, k, alpha, beta, _p(a), k, _p(b), n, _p(out), n, threads)
    if rc != 0:
        raise ValueError("orc_matmul_q8_kmajor: InvalidArgument")
    return out


def matmul_q_packed(dtype, a, b_blocks, n, alpha=1.0, beta=0.0, c=None, kc=256, threads=1):
    a = _f32(a); m, k = a.shape
    b = np.ascontiguousarray(b_blocks, dtype=np.uint8)
    out = _c_init(m, n, c, beta)
    rc = _lib.orc_matmul_q_packed(dtype, m, n, k, alpha, beta, _p(a), k, _p(b), _p(out), n, kc, threads)
    if rc != 0:
        raise ValueError("orc_matmul_q_packed: InvalidArgument")
    return out


def matmul_q_f32a(dtype, nt, a, b_blocks, n, alpha=1.0, beta=0.0, c=None, threads=1):
    a = _f32(a); m, k = a.shape
    b = np.ascontiguousarray(b_blocks, dtype=np.uint8)
    out = _c_init(m, n, c, beta)
    rc = _lib.orc_matmul_q_f32a(dtype, 1 if nt else 0, m, n, k, alpha, beta, _p(a), k, _p(b), _p(out), n, threads)
    if rc != 0:
        raise ValueError("orc_matmul_q_f32a: InvalidArgument")
    return out


class _AttnShape(C.Structure):
    _fields_ = [(n, C.c_size_t) for n in ("batch", "l_q", "t_kv", "h_q", "h_kv", "d_k", "d_v")] + [
        ("scale", C.c_float), ("soft_cap", C.c_float),
        ("win_left", C.c_uint32), ("win_right", C.c_uint32), ("win_chunk", C.c_uint32),
        ("kv_dtype", C.c_int)]


def _attn_args(q, k, v, scale, window, soft_cap, positions, kv_lengths):
    q = _f32(q)
    B, L, Hq, Dk = q.shape
    if k.dtype == np.float16:
        k = np.ascontiguousarray(k).view(np.uint16); v = np.ascontiguousarray(v).view(np.uint16); kvd = 1
    elif k.dtype == np.uint16:
        k = np.ascontiguousarray(k); v = np.ascontiguousarray(v); kvd = 1
    else:
        k = _f32(k); v = _f32(v); kvd = 0
    _, T, Hkv, _ = k.shape
    Dv = v.shape[3]
    left, right, chunk = window
    s = _AttnShape(B, L, T, Hq, Hkv, Dk, Dv, scale, soft_cap, left, right, chunk, kvd)
    pos = None if positions is None else np.ascontiguousarray(positions, dtype=np.int32)
    kl = None if kv_lengths is None else np.ascontiguousarray(kv_lengths, dtype=np.int32)
    out = np.zeros((B, L, Hq, Dv), dtype=np.float32)
    return s, q, k, v, pos, kl, out


CAUSAL = (UNBOUNDED, 0, 0)
FULL = (UNBOUNDED, UNBOUNDED, 0)


def attention_blocked(q, k, v, scale, window=CAUSAL, soft_cap=0.0, positions=None, kv_lengths=None, segs=1):
    s, q, k, v, pos, kl, out = _attn_args(q, k, v, scale, window, soft_cap, positions, kv_lengths)
    rc = _lib.orc_attention_blocked(C.byref(s), _p(q), _p(k), _p(v), _p(pos), _p(kl), _p(out), segs)
    if rc != 0:
        raise ValueError("orc_attention_blocked: InvalidArgument")
    return out


def attention_f64(q, k, v, scale, window=CAUSAL, soft_cap=0.0, positions=None, kv_lengths=None):
    s, q, k, v, pos, kl, out = _attn_args(q, k, v, scale, window, soft_cap, positions, kv_lengths)
    rc = _lib.orc_attention_f64(C.byref(s), _p(q), _p(k), _p(v), _p(pos), _p(kl), _p(out))
    if rc != 0:
        raise ValueError("orc_attention_f64: InvalidArgument")
    return out


def window_keys(window, pos, end):
    """AttentionWindow.keys (graph/graph.zig:160-167): the key interval [lo, hi) of a query at `pos` over keys [0, end)."""
    left, right, chunk = window
    anchor = (pos // chunk) * chunk if chunk > 0 else pos
    span = chunk if chunk > 0 else 1
    lo = anchor - min(anchor, left)
    hi = end if right == UNBOUNDED else min(end, anchor + span + right)
    return lo, max(hi, lo)


def attention_rolling_f64(q, k_ring, v_ring, scale, window, positions, kv_lengths, soft_cap=0.0):
    """Attention over rolling caches, the reference's generic path in f64 (cpu/exec/attention.zig:1055-1160, 1537-1546):
    the cache length may exceed the capacity T; keys older than length - T are gone (:1072-1075); logical key t is
    read from row t % T (:1150-1152). Plain loops: small cases only.
    Pinned in tests/test_oracle_rolling.py by: ring == the unrolled linear cache through orc_attention_f64 whenever
    the window stays inside the retained keys, and ring == the linear cache with its overwritten prefix cut off
    (positions shifted) when it does not."""
    q = np.asarray(q, np.float64)
    k = np.asarray(k_ring, np.float64); v = np.asarray(v_ring, np.float64)
    B, L, Hq, _ = q.shape
    T, Hkv = k.shape[1], k.shape[2]
    out = np.zeros((B, L, Hq, v.shape[3]), np.float64)
    for b in range(B):
        end = int(kv_lengths[b])
        start = max(0, end - T)
        for l in range(L):
            lo, hi = window_keys(window, int(positions[b, l]), end)
            lo = max(lo, start)
            if hi <= lo:
                continue
            rows = np.arange(lo, hi) % T
            for h in range(Hq):
                hk = h // (Hq // Hkv)
                sc = (k[b, rows, hk] @ q[b, l, h]) * scale
                if soft_cap > 0:
                    sc = soft_cap * np.tanh(sc / soft_cap)
                p = np.exp(sc - sc.max())
                out[b, l, h] = (p / p.sum()) @ v[b, rows, hk]
    return out.astype(np.float32)


def sequence_append(cache, new, end_index, rolling=False):
    """StepSequenceAppend (cpu/exec/sequence_append.zig:58-104): rows new[b, s] go to cache[b, map(end_index[b] + s)];
    map is the identity (out of range = InvalidArgument) or t % T for a rolling cache (storage/cache.zig:187-207)."""
    out = np.array(cache, copy=True)
    T = out.shape[1]
    for b in range(out.shape[0]):
        for s_ in range(new.shape[1]):
            t = int(end_index[b]) + s_
            if t < 0 or (not rolling and t >= T):
                raise ValueError("sequence_append: InvalidArgument")
            out[b, t % T if rolling else t] = new[b, s_]
    return out


def grow_target(current, num, den):
    """StorageManager.growTarget (storage/manager.zig:69-76; the same rule as storage/cache.zig:129-137)."""
    if current == 0 or num == 0 or den == 0:
        raise ValueError("grow_target: InvalidArgument")
    nxt = (current * num + den - 1) // den
    return current + 1 if nxt <= current else nxt


def grow_axis(cache, axis, new_size):
    """growAxisOnDevice / growAxisPreserveScalar (storage/manager/grow.zig:37-78): the tensor grows along `axis`, existing
    elements keep their indices, new elements are zero."""
    cache = np.asarray(cache)
    if new_size < cache.shape[axis]:
        raise ValueError("grow_axis: InvalidArgument")
    shape = list(cache.shape)
    shape[axis] = new_size
    out = np.zeros(shape, cache.dtype)
    out[tuple(slice(0, n) for n in cache.shape)] = cache
    return out


def grow_rolling(cache, new_capacity, retained_history, logical_ends):
    """ensureRollingCacheCapacity (storage/manager/grow.zig:107-150): cache [B, T, ...] is a ring; the last
    min(end, retained_history, T) logical steps before each batch entry's end move to row t % new_capacity, the rest
    of the new ring is zero."""
    cache = np.asarray(cache)
    B, T = cache.shape[0], cache.shape[1]
    if len(logical_ends) != B or T == 0:
        raise ValueError("grow_rolling: InvalidArgument")
    if T >= new_capacity:
        return cache.copy()
    out = np.zeros((B, new_capacity) + cache.shape[2:], cache.dtype)
    for b, end in enumerate(logical_ends):
        end = int(end)
        kept = min(end, retained_history, T)
        for t in range(end - kept, end):
            out[b, t % new_capacity] = cache[b, t % T]
    return out


def session_growth_target(capacity, required, num, den, max_capacity=0):
    """growSequenceCache (api/loaded_model.zig:791-827): geometric steps until `required` fits, then rounded up to a
    power of two and to at least four times the old capacity (each capacity is a compiled shape), clipped to the
    policy's ceiling. Rolling caches use the factor 2/1 and no ceiling."""
    target = capacity
    while target < required:
        target = grow_target(target, num, den)
    p2 = 1
    while p2 < target:
        p2 *= 2
    target = max(p2, capacity * 4)
    if max_capacity:
        if required > max_capacity:
            raise ValueError("session_growth_target: InvalidArgument")
        target = min(target, max_capacity)
    return target


def rmsnorm(x, gamma, eps, beta=None, residual=None):
    x = _f32(x); rows, cols = x.shape
    g = _f32(gamma); b = None if beta is None else _f32(beta); r = None if residual is None else _f32(residual)
    out = np.zeros_like(x)
    _lib.orc_rmsnorm(_p(x), _p(g), _p(b), _p(r), rows, cols, eps, _p(out))
    return out


def rope(x, positions, base=10000.0, scale_factor=1.0, proportion=1.0):
    x = _f32(x); B, T, H, D = x.shape
    pos = np.ascontiguousarray(positions, dtype=np.int32)
    out = np.zeros_like(x)
    _lib.orc_rope(_p(x), _p(pos), B, T, H, D, base, scale_factor, proportion, _p(out))
    return out


def gate_gelu(a, b):
    a = _f32(a); b = _f32(b)
    out = np.zeros_like(a)
    _lib.orc_gate_gelu(_p(a), _p(b), a.size, _p(out))
    return out


UNARY_OPS = {"relu": 0, "gelu": 1, "silu": 2, "sigmoid": 3, "tanh": 4, "sqrt": 5}
BINARY_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3}


def unary(op, x):
    x = _f32(x)
    out = np.zeros_like(x)
    if _lib.orc_unary(UNARY_OPS[op], _p(x), x.size, _p(out)):
        raise ValueError("orc_unary: InvalidArgument")
    return out


def binary(op, a, b):
    """b has a's shape, one element, or a contiguous suffix of a's shape."""
    a = _f32(a); b = _f32(b)
    out = np.zeros_like(a)
    if _lib.orc_binary(BINARY_OPS[op], _p(a), _p(b), a.size, b.size, _p(out)):
        raise ValueError("orc_binary: InvalidArgument")
    return out


def gather_rows(table, ids, d, dtype=0):
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    t = np.ascontiguousarray(table)
    out = np.zeros((ids.size, d), dtype=np.float32)
    _lib.orc_gather_rows(dtype, _p(t), d, _p(ids), ids.size, _p(out))
    return out


def argmax(x):
    x = _f32(x); rows, n = x.shape
    out = np.zeros(rows, dtype=np.int32)
    _lib.orc_argmax(_p(x), rows, n, _p(out))
    return out


def cast_f32_f16(x):
    x = _f32(x)
    out = np.zeros(x.shape, dtype=np.uint16)
    _lib.orc_cast_f32_f16(_p(x), x.size, _p(out))
    return out.view(np.float16)


class _DecCfg(C.Structure):
    _fields_ = [(n, C.c_size_t) for n in ("layers", "hidden", "heads", "kv_heads", "head_dim", "ffn", "vocab", "max_seq")] + [
        ("eps", C.c_float), ("rope_base", C.c_float), ("wdtype", C.c_int), ("attn_exact", C.c_int)]


class Decoder:
    """The synthetic decoder run through the oracle kernels (see orc_decoder_* in aion_oracle.h)."""

    def __init__(self, layers, hidden, heads, kv_heads, head_dim, ffn, vocab, max_seq,
                 eps=1e-6, rope_base=10000.0, wdtype=Q4_0, threads=1, attn_exact=False):
        self.cfg = _DecCfg(layers, hidden, heads, kv_heads, head_dim, ffn, vocab, max_seq, eps, rope_base, wdtype, 1 if attn_exact else 0)
        self.vocab = vocab
        self._h = _lib.orc_decoder_create(C.byref(self.cfg), threads)

    def set_weight(self, name, data):
        d = np.ascontiguousarray(data)
        _lib.orc_decoder_set_weight(self._h, name.encode(), _p(d), d.nbytes)

    def reset(self):
        _lib.orc_decoder_reset(self._h)

    def forward(self, tokens, pos0, want_logits=True):
        t = np.ascontiguousarray(tokens, dtype=np.int32)
        logits = np.zeros(self.vocab, dtype=np.float32) if want_logits else None
        tok = _lib.orc_decoder_forward(self._h, _p(t), t.size, pos0, _p(logits))
        if tok < 0:
            raise ValueError("orc_decoder_forward failed")
        return int(tok), logits

    def __del__(self):
        if getattr(self, "_h", None):
            _lib.orc_decoder_destroy(self._h)
            self._h = None
