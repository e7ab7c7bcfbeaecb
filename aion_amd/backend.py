"""Host-side mirror of aion's backend vocabulary over the C ABI (numpy in, numpy out).

Names follow aion: a `HipBackend` owns one device context (Backend + Session,
backend/backend.zig:24-107), `DeviceBuffer` is a DeviceMemory allocation
(runtime/device_memory.zig:36-108), `Weight` is a quantized rank-2 parameter after the
backend's private re-lay, and the `step_*` methods take the operands of the matching
ExecutableProgram step (runtime/executable.zig).
"""
import ctypes as C

import numpy as np

from . import hip
from .hip import (BF16, F16, F32, GEMM_BF16_MFMA, GEMM_BF16_MFMA_ALWAYS, GEMM_EXACT_I8, I32, KMAJOR_KN, Q4_0, Q8_0, ROWS_NK, UNBOUNDED,  # noqa: F401
                  AionHipError)

BLOCK_BYTES = {Q4_0: 18, Q8_0: 34}
CAUSAL = (UNBOUNDED, 0, 0)
FULL = (UNBOUNDED, UNBOUNDED, 0)


def quantize_blocks(dtype, values, quant_axis):
    """storage/quantize.zig `quantizeBlocks` over the whole tensor: f32 array -> packed bytes."""
    lib = hip.load_library()
    v = np.ascontiguousarray(values, dtype=np.float32)
    if v.ndim == 0:
        raise AionHipError(hip.INVALID_ARGUMENT, "rank-0 tensor")
    if dtype not in BLOCK_BYTES:
        raise AionHipError(hip.UNSUPPORTED, "dtype %r is not block-quantized" % (dtype,))
    shape = (C.c_size_t * v.ndim)(*v.shape)
    out = np.empty(v.size // 32 * BLOCK_BYTES[dtype], dtype=np.uint8)
    rc = lib.aionhip_quantize_blocks(dtype, shape, v.ndim, quant_axis, v.ctypes.data, v.size, 0, 0, out.ctypes.data, out.nbytes)
    if rc != hip.OK:
        raise AionHipError(rc, "quantize_blocks(shape=%s, axis=%d)" % (v.shape, quant_axis))
    return out


class DeviceBuffer:
    def __init__(self, backend, handle, nbytes):
        self.backend, self.handle, self.nbytes = backend, handle, nbytes

    def free(self):
        if self.handle:
            self.backend._lib.aionhip_free(self.backend._ctx, self.handle)
            self.handle = 0

    def numpy(self, dtype, shape=None, offset=0):
        return self.backend.download(self, dtype, shape, offset)

    def view(self, offset_bytes):
        """A non-owning window starting `offset_bytes` into this allocation."""
        v = DeviceBuffer(self.backend, self.handle + offset_bytes, self.nbytes - offset_bytes)
        v.free = lambda: None
        return v


class Weight:
    def __init__(self, backend, ptr, dtype, layout, n, k):
        self.backend, self.ptr, self.dtype, self.layout, self.n, self.k = backend, ptr, dtype, layout, n, k

    @property
    def packed_bytes(self):
        return self.backend._lib.aionhip_weight_packed_bytes(self.ptr)

    @property
    def device_bytes(self):
        return self.backend._lib.aionhip_weight_device_bytes(self.ptr)

    def download(self):
        out = np.empty(self.packed_bytes, dtype=np.uint8)
        self.backend._check(self.backend._lib.aionhip_weight_download(self.backend._ctx, self.ptr, out.ctypes.data, out.nbytes))
        return out

    def drop_bf16(self):
        """Releases the bf16 copy the context keeps of this weight in bf16 GEMM mode (rebuilt on its next bf16 call)."""
        if self.ptr:
            self.backend._lib.aionhip_weight_drop_bf16(self.backend._ctx, self.ptr)

    def free(self):
        if self.ptr:
            self.backend._lib.aionhip_weight_free(self.backend._ctx, self.ptr)
            self.ptr = None


class HipBackend:
    def __init__(self, device=0, stream=None):
        self._lib = hip.load_library()
        ctx = C.c_void_p()
        rc = self._lib.aionhip_create(device, stream, C.byref(ctx))
        if rc != hip.OK:
            raise AionHipError(rc, "aionhip_create(device=%d): no usable HIP device" % device)
        self._ctx = ctx
        self.name = self._lib.aionhip_name().decode()

    # ---- context
    def _check(self, rc):
        if rc != hip.OK:
            raise AionHipError(rc, self._lib.aionhip_last_error(self._ctx).decode())

    def close(self):
        if self._ctx:
            self._lib.aionhip_destroy(self._ctx)
            self._ctx = None

    def sync(self):
        self._check(self._lib.aionhip_sync(self._ctx))

    def last_kernel(self):
        return self._lib.aionhip_last_kernel(self._ctx).decode()

    def last_launch(self):
        """The last launch a step made: {"kernel": instance name as a kernel trace prints it, "grid", "block", "lds"}."""
        name = C.create_string_buffer(512)
        grid, block, lds = (C.c_uint * 3)(), (C.c_uint * 3)(), C.c_size_t()
        self._check(self._lib.aionhip_last_launch(self._ctx, name, len(name), grid, block, C.byref(lds)))
        return {"kernel": name.value.decode(), "grid": list(grid), "block": list(block), "lds": int(lds.value)}

    def set_gemm_mode(self, mode):
        self._check(self._lib.aionhip_set_gemm_mode(self._ctx, mode))

    def set_attention_precise(self, on):
        self._check(self._lib.aionhip_set_attention_precise(self._ctx, 1 if on else 0))

    def device_info(self):
        cu, wave, hbm = C.c_int(), C.c_int(), C.c_uint64()
        arch = C.create_string_buffer(64)
        self._check(self._lib.aionhip_device_info(self._ctx, C.byref(cu), C.byref(wave), C.byref(hbm), arch, 64))
        return {"cu_count": cu.value, "wave_size": wave.value, "hbm_bytes": hbm.value, "arch": arch.value.decode()}

    # ---- device memory
    def alloc(self, nbytes, alignment=256):
        h = C.c_uint64()
        self._check(self._lib.aionhip_alloc(self._ctx, nbytes, alignment, C.byref(h)))
        return DeviceBuffer(self, h.value, nbytes)

    def trim(self):
        """Gives the blocks the context's pool has cached back to the device (waits for the stream)."""
        self._check(self._lib.aionhip_trim(self._ctx))

    def memory_stats(self):
        """(bytes handed out by alloc and not yet freed, bytes of freed blocks the pool keeps for reuse)"""
        live, cached = C.c_uint64(), C.c_uint64()
        self._check(self._lib.aionhip_memory_stats(self._ctx, C.byref(live), C.byref(cached)))
        return live.value, cached.value

    def upload(self, array):
        a = np.ascontiguousarray(array)
        buf = self.alloc(max(a.nbytes, 1))
        if a.nbytes:
            self._check(self._lib.aionhip_h2d(self._ctx, buf.handle, 0, a.ctypes.data, a.nbytes))
        return buf

    def write(self, buf, array, offset=0):
        a = np.ascontiguousarray(array)
        self._check(self._lib.aionhip_h2d(self._ctx, buf.handle, offset, a.ctypes.data, a.nbytes))

    def download(self, buf, dtype, shape=None, offset=0):
        dt = np.dtype(dtype)
        if shape is None:
            shape = ((buf.nbytes - offset) // dt.itemsize,)
        out = np.empty(shape, dtype=dt)
        if out.nbytes:
            self._check(self._lib.aionhip_d2h(self._ctx, out.ctypes.data, buf.handle, offset, out.nbytes))
        return out

    def copy(self, dst, src, nbytes, dst_offset=0, src_offset=0):
        """DeviceMemory.copyD2D on the context's stream (asynchronous)."""
        self._check(self._lib.aionhip_d2d(self._ctx, dst.handle, dst_offset, src.handle, src_offset, nbytes))

    def zeros(self, nbytes):
        buf = self.alloc(nbytes)
        self._check(self._lib.aionhip_memset(self._ctx, buf.handle, 0, 0, nbytes))
        return buf

    # ---- quantize / weights
    def quantize_device(self, dtype, src_buf, rows, cols, quant_axis):
        out = self.alloc(rows * cols // 32 * BLOCK_BYTES[dtype])
        self._check(self._lib.aionhip_quantize_device(self._ctx, dtype, rows, cols, quant_axis, src_buf.handle, out.handle))
        return out

    def upload_weight(self, dtype, layout, n, k, packed_blocks, ld_blocks=0):
        if dtype == F32:          # the f32 [N,K] operand of MatMulNT: the rows as they are
            b = np.ascontiguousarray(packed_blocks, dtype=np.float32).reshape(-1).view(np.uint8)
        else:
            b = np.ascontiguousarray(packed_blocks, dtype=np.uint8)
        w = C.c_void_p()
        self._check(self._lib.aionhip_weight_upload(self._ctx, dtype, layout, n, k, ld_blocks, b.ctypes.data, C.byref(w)))
        return Weight(self, w, dtype, layout, n, k)

    def weight_from_device(self, dtype, layout, n, k, blocks_buf, ld_blocks=0):
        w = C.c_void_p()
        self._check(self._lib.aionhip_weight_from_device(self._ctx, dtype, layout, n, k, ld_blocks, blocks_buf.handle, C.byref(w)))
        return Weight(self, w, dtype, layout, n, k)

    # ---- steps
    def step_matmul(self, weight, a_buf, m, c_buf, lda=0, ldc=0, alpha=1.0, beta=0.0, a_offset=0, c_offset=0):
        fn = self._lib.aionhip_step_matmul_nt if weight.layout == ROWS_NK else self._lib.aionhip_step_matmul
        self._check(fn(self._ctx, weight.ptr, m, a_buf.handle + a_offset, lda, c_buf.handle + c_offset, ldc, alpha, beta))

    def step_matmul_static(self, weight, a_buf, m, c_buf, lda=0, ldc=0, alpha=1.0, beta=0.0):
        """step_matmul through the entry point that allocates nothing (prepared activation in the library's static array)."""
        self._check(self._lib.aionhip_step_matmul_static(self._ctx, weight.ptr, m, a_buf.handle, lda, c_buf.handle, ldc, alpha, beta))

    def step_matmul_batch(self, weights, a_buf, m, c_bufs, lda=0, alpha=1.0, beta=0.0, c_offsets=None):
        n = len(weights)
        ws = (C.c_void_p * n)(*[w.ptr.value for w in weights])
        offs = c_offsets or [0] * n
        cs = (C.c_uint64 * n)(*[b.handle + o for b, o in zip(c_bufs, offs)])
        self._check(self._lib.aionhip_step_matmul_batch(self._ctx, n, ws, m, a_buf.handle, lda, cs, None, alpha, beta))

    def step_rmsnorm_matmul(self, weights, x, gamma, rows, c_bufs, eps, beta_norm=None, alpha=1.0, beta=0.0):
        n = len(weights)
        ws = (C.c_void_p * n)(*[w.ptr.value for w in weights])
        cs = (C.c_uint64 * n)(*[b.handle for b in c_bufs])
        self._check(self._lib.aionhip_step_rmsnorm_matmul(self._ctx, n, ws, rows, x.handle, gamma.handle,
                                                          beta_norm.handle if beta_norm is not None else 0, eps, cs, None, alpha, beta))

    def step_gate_matmul(self, weight, gate, up, rows, c_buf, alpha=1.0, beta=0.0):
        self._check(self._lib.aionhip_step_gate_matmul(self._ctx, weight.ptr, rows, gate.handle, up.handle, c_buf.handle, 0, alpha, beta))

    def step_rope_append(self, q_out, q, k, v, k_cache, v_cache, positions, write_index, b, s, t_cap, h_q, h_kv, d,
                         base=10000.0, scale_factor=1.0, proportion=1.0):
        self._check(self._lib.aionhip_step_rope_append(self._ctx, q_out.handle, q.handle, k.handle, v.handle, k_cache.handle, v_cache.handle,
                                                       positions.handle, write_index.handle, b, s, t_cap, h_q, h_kv, d, base, scale_factor, proportion))

    def step_rmsnorm_qkv_rope_append(self, wq, wk, wv, x, gamma, eps, q_out, k_cache, v_cache, positions, write_index,
                                     t_cap, h_q, h_kv, d, base=10000.0, scale_factor=1.0, proportion=1.0, beta_norm=None, rolling=False):
        """One new token of one sequence: RMSNorm -> q/k/v matmuls -> RoPE -> f16 cache append (rolling: into rings), one launch."""
        self._check(self._lib.aionhip_step_rmsnorm_qkv_rope_append(
            self._ctx, wq.ptr, wk.ptr, wv.ptr, x.handle, gamma.handle, beta_norm.handle if beta_norm is not None else 0, eps,
            q_out.handle, k_cache.handle, v_cache.handle, positions.handle, write_index.handle, t_cap, h_q, h_kv, d,
            base, scale_factor, proportion, 1 if rolling else 0))

    def step_rmsnorm_geglu_matmul(self, w_gate, w_up, w_down, x, gamma, eps, c_buf, alpha=1.0, beta=0.0, beta_norm=None):
        """One activation row: RMSNorm -> gate/up matmuls -> gelu gate -> down matmul, two launches."""
        self._check(self._lib.aionhip_step_rmsnorm_geglu_matmul(
            self._ctx, w_gate.ptr, w_up.ptr, w_down.ptr, x.handle, gamma.handle, beta_norm.handle if beta_norm is not None else 0, eps,
            c_buf.handle, alpha, beta))

    # ---- a run of decoder blocks as one launch (one new token of one sequence)
    def decoder_stack_create(self, layers, hidden, heads, kv_heads, head_dim, ffn, t_cap, eps1, eps2, attn_scale, rope_base=10000.0,
                             rope_scale=1.0, rope_proportion=1.0, soft_cap=0.0, window=CAUSAL, rolling=False):
        """layers: one dict per block with the weights wq, wk, wv, wo, w_gate, w_up, w_down (Weight), norm1_gamma, norm2_gamma,
        k_cache, v_cache (DeviceBuffer) and optionally norm1_beta, norm2_beta. Raises AionHipError(UNSUPPORTED) for shapes the
        one-launch form does not take."""
        desc = hip.DecoderStackDesc(len(layers), hidden, heads, kv_heads, head_dim, ffn, t_cap, eps1, eps2, rope_base, rope_scale,
                                    rope_proportion, attn_scale, soft_cap, window[0], window[1], window[2], 1 if rolling else 0)
        arr = (hip.DecoderStackLayer * len(layers))()
        for i, l in enumerate(layers):
            for name in ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down"):
                setattr(arr[i], name, l[name].ptr)
            for name in ("norm1_gamma", "norm1_beta", "norm2_gamma", "norm2_beta", "k_cache", "v_cache"):
                buf = l.get(name)
                setattr(arr[i], name, buf.handle if buf is not None else 0)
        st = C.c_void_p()
        self._check(self._lib.aionhip_decoder_stack_create(self._ctx, C.byref(desc), arr, C.byref(st)))
        return st

    def decoder_stack_destroy(self, stack):
        self._lib.aionhip_decoder_stack_destroy(self._ctx, stack)

    def step_decoder_stack(self, stack, x_in, x_out, positions, write_index, kv_lengths):
        self._check(self._lib.aionhip_step_decoder_stack(self._ctx, stack, x_in.handle, x_out.handle, positions.handle, write_index.handle,
                                                         kv_lengths.handle))

    def decoder_stack_status(self, stack):
        """Waits for the stream; raises AionHipError(EXECUTION_FAILED) if a launch of the stack gave up waiting since the last call."""
        failed = C.c_int(0)
        self._check(self._lib.aionhip_decoder_stack_status(self._ctx, stack, C.byref(failed)))

    def decoder_stack_set_stamps(self, stack, buf):
        """Time stamps of the next launches into `buf` (2 x layers x 10 counters of 8 bytes, 100 MHz), None switches them off."""
        self._check(self._lib.aionhip_decoder_stack_set_stamps(self._ctx, stack, buf.handle if buf is not None else 0))

    def decoder_stack_set_poll_budget(self, stack, milliseconds):
        self._check(self._lib.aionhip_decoder_stack_set_poll_budget(self._ctx, stack, float(milliseconds)))

    def step_add_i32(self, out, a, b, n):
        self._check(self._lib.aionhip_step_add_i32(self._ctx, out.handle, a.handle, b.handle, n))

    def step_advance_state(self, dst_tokens, src_tokens, n_tokens, counters, delta=1, log=None, log_index=None, log_capacity=0):
        """One launch: dst_tokens <- src_tokens (i32) and delta added to every scalar i32 buffer in `counters`; with `log`,
        the tokens also go to log[*log_index ..] (the index is read before the counters move and may be one of them)."""
        n = len(counters)
        arr = (C.c_uint64 * max(n, 1))(*[c.handle for c in counters])
        if log is None:
            self._check(self._lib.aionhip_step_advance_state(self._ctx, dst_tokens.handle, src_tokens.handle, n_tokens, arr, n, delta))
        else:
            self._check(self._lib.aionhip_step_advance_state_log(self._ctx, dst_tokens.handle, src_tokens.handle, n_tokens, arr, n, delta,
                                                                 log.handle, log_index.handle, log_capacity))

    # ---- programs (HIP graph replay of a recorded step sequence)
    def program_begin(self):
        self._check(self._lib.aionhip_program_begin(self._ctx))

    def program_end(self):
        p = C.c_void_p()
        self._check(self._lib.aionhip_program_end(self._ctx, C.byref(p)))
        return p

    def program_abort(self):
        self._check(self._lib.aionhip_program_abort(self._ctx))

    def record_program(self, issue):
        """Records the steps `issue()` makes into a program. If a step raises, the recording is dropped (the context is
        left executing eagerly, not stuck in capture) and the error propagates."""
        self.program_begin()
        try:
            issue()
        except BaseException:
            self._lib.aionhip_program_abort(self._ctx)
            raise
        return self.program_end()

    def program_execute(self, prog):
        self._check(self._lib.aionhip_program_execute(self._ctx, prog))

    def set_bf16_weight_copies(self, on):
        """bf16 GEMM mode: True (default) keeps a bf16 copy per weight, False converts the quant blocks inside the kernel."""
        self._check(self._lib.aionhip_set_bf16_weight_copies(self._ctx, 1 if on else 0))

    def bf16_copy_stats(self):
        n, b = C.c_uint64(0), C.c_uint64(0)
        self._check(self._lib.aionhip_bf16_copy_stats(self._ctx, C.byref(n), C.byref(b)))
        return n.value, b.value

    def program_is_current(self, prog):
        """False once a work buffer the program's launches address has been replaced by a larger one: record it again."""
        return bool(self._lib.aionhip_program_is_current(self._ctx, prog))

    def program_node_count(self, prog):
        return self._lib.aionhip_program_node_count(prog)

    def program_destroy(self, prog):
        self._lib.aionhip_program_destroy(self._ctx, prog)

    def matmul(self, weight, a, alpha=1.0, beta=0.0, c=None):
        """Convenience: numpy A [m,k] -> numpy C [m,n] through the step (uploads, runs, downloads)."""
        a = np.ascontiguousarray(a, dtype=np.float32)
        m = a.shape[0]
        a_buf = self.upload(a)
        if c is None:
            c_buf = self.alloc(max(m * weight.n * 4, 4))
        else:
            c_buf = self.upload(np.ascontiguousarray(c, dtype=np.float32))
        try:
            self.step_matmul(weight, a_buf, m, c_buf, alpha=alpha, beta=beta)
            return self.download(c_buf, np.float32, (m, weight.n))
        finally:
            a_buf.free()
            c_buf.free()

    def step_attention(self, out, q, k, v, shape, scale, q_dtype=F32, kv_dtype=F16, window=CAUSAL, soft_cap=0.0,
                       query_positions=None, kv_lengths=None, rolling=False):
        B, L, T, Hq, Hkv, Dk, Dv = shape
        p = hip.Attention(out.handle, q.handle, k.handle, v.handle,
                          query_positions.handle if query_positions is not None else 0,
                          kv_lengths.handle if kv_lengths is not None else 0,
                          B, L, T, Hq, Hkv, Dk, Dv, q_dtype, kv_dtype, scale, soft_cap, window[0], window[1], window[2],
                          1 if rolling else 0)
        self._check(self._lib.aionhip_step_attention(self._ctx, C.byref(p)))

    def step_rmsnorm(self, out, x, gamma, rows, cols, eps, beta=None, residual=None):
        self._check(self._lib.aionhip_step_rmsnorm(self._ctx, out.handle, x.handle, gamma.handle,
                                                   beta.handle if beta is not None else 0,
                                                   residual.handle if residual is not None else 0, rows, cols, eps))

    def step_rope(self, out, x, positions, b, t, h, d, base=10000.0, scale_factor=1.0, proportion=1.0):
        self._check(self._lib.aionhip_step_rope(self._ctx, out.handle, x.handle, positions.handle, b, t, h, d, base, scale_factor, proportion))

    def step_add(self, out, a, b, n):
        self._check(self._lib.aionhip_step_add(self._ctx, out.handle, a.handle, b.handle, n))

    def step_gate_gelu(self, out, a, b, n):
        self._check(self._lib.aionhip_step_gate_gelu(self._ctx, out.handle, a.handle, b.handle, n))

    def step_gather_rows(self, table_dtype, out, table, ids, n_ids, d, vocab):
        self._check(self._lib.aionhip_step_gather_rows(self._ctx, table_dtype, out.handle, table.handle, ids.handle, n_ids, d, vocab))

    def step_append_f16(self, cache, src, write_index, b, s, t_cap, row_elems, rolling=False):
        self._check(self._lib.aionhip_step_append_f16(self._ctx, cache.handle, src.handle, write_index.handle, b, s, t_cap, row_elems,
                                                      1 if rolling else 0))

    def step_sequence_append(self, dtype, cache, new_kv, end_index, b, s, t_cap, row_elems, rolling=False):
        """StepSequenceAppend with rows and cache of one element type, F16 or F32 (cpu/exec/sequence_append.zig:12-104)."""
        self._check(self._lib.aionhip_step_sequence_append(self._ctx, dtype, cache.handle, new_kv.handle, end_index.handle, b, s, t_cap,
                                                           row_elems, 1 if rolling else 0))

    def cache_grow(self, dst, src, outer, old_run_bytes, new_run_bytes):
        """dst [outer, new_run_bytes] <- the runs of src [outer, old_run_bytes], zero elsewhere (storage/manager/grow.zig:37-78)."""
        self._check(self._lib.aionhip_cache_grow(self._ctx, dst.handle, src.handle, outer, old_run_bytes, new_run_bytes))

    def cache_grow_rolling(self, dst, src, logical_ends, b, old_capacity, new_capacity, row_bytes, retained_history):
        """Ring growth: the retained logical steps move to row t % new_capacity (storage/manager/grow.zig:107-150)."""
        self._check(self._lib.aionhip_cache_grow_rolling(self._ctx, dst.handle, src.handle, logical_ends.handle, b, old_capacity,
                                                         new_capacity, row_bytes, retained_history))

    def cache_grow_target(self, current, num, den):
        """Next capacity of the geometric schedule (storage/manager.zig:69-76); raises on invalid arguments."""
        t = int(self._lib.aionhip_cache_grow_target(current, num, den))
        if t == 0:
            raise ValueError("cache_grow_target: InvalidArgument")
        return t

    UNARY = {"relu": 0, "gelu": 1, "silu": 2, "sigmoid": 3, "tanh": 4, "sqrt": 5, "log": 6}
    BINARY = {"add": 0, "sub": 1, "mul": 2, "div": 3}

    def step_unary(self, op, out, x, n):
        """StepUnary on f32; op by aion's name (backend/types.zig:119-128)."""
        self._check(self._lib.aionhip_step_unary(self._ctx, self.UNARY[op], out.handle, x.handle, n))

    def step_binary(self, op, out, a, b, n, nb=None):
        """StepElemwiseBinary add/sub/mul/div on f32: out[i] = a[i] op b[i % nb] (nb = n: same shape; 1: scalar)."""
        self._check(self._lib.aionhip_step_binary(self._ctx, self.BINARY[op], out.handle, a.handle, b.handle, n, n if nb is None else nb))

    def step_headnorm_rope_append(self, q_out, q, k, v, gammas, betas, eps, k_cache, v_cache, positions, write_index, b, s, t_cap,
                                  h_q, h_kv, d, base=10000.0, scale_factor=1.0, proportion=1.0, rolling=False):
        """Per-head RMSNorm on q, k, v (gammas / betas: three buffers each, a beta may be None) -> RoPE(q, k) -> f16
        cache append of k and v, one launch."""
        hb = [x.handle if x is not None else 0 for x in betas]
        self._check(self._lib.aionhip_step_headnorm_rope_append(
            self._ctx, q_out.handle, q.handle, k.handle, v.handle, gammas[0].handle, hb[0], gammas[1].handle, hb[1], gammas[2].handle, hb[2],
            eps, k_cache.handle, v_cache.handle, positions.handle, write_index.handle, b, s, t_cap, h_q, h_kv, d, base, scale_factor,
            proportion, 1 if rolling else 0))

    def step_cast_f32_f16(self, out, x, n):
        self._check(self._lib.aionhip_step_cast_f32_f16(self._ctx, out.handle, x.handle, n))

    def probe_stream_read(self, src, offset, nbytes, sink):
        """Plain streaming read of nbytes of src (measurement aid; profiled as "stream_read")."""
        self._check(self._lib.aionhip_probe_stream_read(self._ctx, src.handle, offset, nbytes, sink.handle))

    def step_argmax(self, out, x, rows, n):
        self._check(self._lib.aionhip_step_argmax(self._ctx, out.handle, x.handle, rows, n))

    # ---- timing
    def event(self):
        e = C.c_void_p()
        self._check(self._lib.aionhip_event_create(self._ctx, C.byref(e)))
        return e

    def record(self, e):
        self._check(self._lib.aionhip_event_record(self._ctx, e))

    def elapsed_ms(self, start, stop):
        ms = C.c_float()
        self._check(self._lib.aionhip_event_elapsed_ms(self._ctx, start, stop, C.byref(ms)))
        return ms.value

    def profile_start(self):
        self._check(self._lib.aionhip_profile_start(self._ctx))

    def profile_stop(self):
        """-> list of (kernel name, milliseconds), one per timed launch, in launch order."""
        n = C.c_size_t()
        self._check(self._lib.aionhip_profile_stop(self._ctx, C.byref(n)))
        out = []
        name, ms = C.c_char_p(), C.c_float()
        for i in range(n.value):
            self._check(self._lib.aionhip_profile_entry(self._ctx, i, C.byref(name), C.byref(ms)))
            out.append((name.value.decode(), ms.value))
        return out
