"""ctypes binding of libaion_hip.so (include/aion_hip.h). No CPU fallback: a missing or
unloadable library is an error."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libaion_hip.so")

OK, INVALID_ARGUMENT, OUT_OF_MEMORY, UNSUPPORTED, EXECUTION_FAILED = range(5)
STATUS_NAMES = {0: "OK", 1: "InvalidArgument", 2: "OutOfMemory", 3: "Unsupported", 4: "ExecutionFailed"}
F32, F16, I8, Q4_0, Q8_0, I32, BF16 = 0, 1, 2, 3, 4, 5, 16
ROWS_NK, KMAJOR_KN = 0, 1
GEMM_EXACT_I8, GEMM_BF16_MFMA, GEMM_BF16_MFMA_ALWAYS = 0, 1, 2
UNBOUNDED = 0xFFFFFFFF
STATIC_SCRATCH_BYTES = 1 << 20     # AIONHIP_STATIC_SCRATCH_BYTES


class AionHipError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("%s: %s" % (STATUS_NAMES.get(status, status), message))
        self.status = status


class Attention(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in ("out", "q", "k", "v", "query_positions", "kv_lengths")] + \
               [(n, C.c_size_t) for n in ("batch", "l_q", "t_kv", "h_q", "h_kv", "d_k", "d_v")] + \
               [("q_dtype", C.c_int), ("kv_dtype", C.c_int), ("scale", C.c_float), ("attn_logits_soft_cap", C.c_float),
                ("window_left", C.c_uint32), ("window_right", C.c_uint32), ("window_chunk", C.c_uint32), ("rolling", C.c_uint32)]


class DecoderStackLayer(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down")] + \
               [(n, C.c_uint64) for n in ("norm1_gamma", "norm1_beta", "norm2_gamma", "norm2_beta", "k_cache", "v_cache")]


class DecoderStackDesc(C.Structure):
    _fields_ = [(n, C.c_size_t) for n in ("layers", "hidden", "heads", "kv_heads", "head_dim", "ffn", "t_cap")] + \
               [(n, C.c_float) for n in ("eps1", "eps2", "rope_base", "rope_scale", "rope_proportion", "attn_scale", "attn_logits_soft_cap")] + \
               [("window_left", C.c_uint32), ("window_right", C.c_uint32), ("window_chunk", C.c_uint32), ("rolling", C.c_int)]


MAX_RANK = 8


class TensorRef(C.Structure):
    """aionhip_tensor_ref: what the tensor store answers for one TensorId (address, dtype, shape)."""
    _fields_ = [("handle", C.c_uint64), ("dtype", C.c_int32), ("rank", C.c_uint32), ("flags", C.c_uint32), ("reserved", C.c_uint32),
                ("shape", C.c_uint64 * MAX_RANK)]


class Step(C.Structure):
    """aionhip_step: one step of an ExecutableProgram (runtime/executable.zig:302-345) with its operands resolved."""
    _fields_ = [("tag", C.c_int32), ("op", C.c_int32), ("act", C.c_int32), ("broadcast", C.c_int32), ("axis", C.c_int32),
                ("batch_dims", C.c_uint32), ("alpha", C.c_float), ("beta", C.c_float), ("eps", C.c_float), ("scale", C.c_float),
                ("soft_cap", C.c_float), ("window_left", C.c_uint32), ("window_right", C.c_uint32), ("window_chunk", C.c_uint32),
                ("rope_base", C.c_float), ("rope_scale", C.c_float), ("rope_proportion", C.c_float), ("to_host", C.c_int32),
                ("out", TensorRef), ("in_", TensorRef * 5), ("host", C.c_void_p), ("host_bytes", C.c_uint64)]


_SIGS = {
    # name: (restype, argtypes)
    "aionhip_create": (C.c_int, [C.c_int, C.c_void_p, C.POINTER(C.c_void_p)]),
    "aionhip_destroy": (None, [C.c_void_p]),
    "aionhip_sync": (C.c_int, [C.c_void_p]),
    "aionhip_last_error": (C.c_char_p, [C.c_void_p]),
    "aionhip_last_kernel": (C.c_char_p, [C.c_void_p]),
    "aionhip_last_launch": (C.c_int, [C.c_void_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_uint), C.POINTER(C.c_uint), C.POINTER(C.c_size_t)]),
    "aionhip_name": (C.c_char_p, []),
    "aionhip_stream": (C.c_void_p, [C.c_void_p]),
    "aionhip_device_info": (C.c_int, [C.c_void_p, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_uint64), C.c_char_p, C.c_size_t]),
    "aionhip_alloc": (C.c_int, [C.c_void_p, C.c_size_t, C.c_size_t, C.POINTER(C.c_uint64)]),
    "aionhip_free": (None, [C.c_void_p, C.c_uint64]),
    "aionhip_trim": (C.c_int, [C.c_void_p]),
    "aionhip_memory_stats": (C.c_int, [C.c_void_p, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "aionhip_h2d": (C.c_int, [C.c_void_p, C.c_uint64, C.c_size_t, C.c_void_p, C.c_size_t]),
    "aionhip_d2h": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint64, C.c_size_t, C.c_size_t]),
    "aionhip_d2d": (C.c_int, [C.c_void_p, C.c_uint64, C.c_size_t, C.c_uint64, C.c_size_t, C.c_size_t]),
    "aionhip_memset": (C.c_int, [C.c_void_p, C.c_uint64, C.c_size_t, C.c_int, C.c_size_t]),
    "aionhip_quantize_blocks": (C.c_int, [C.c_int, C.POINTER(C.c_size_t), C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t]),
    "aionhip_quantize_device": (C.c_int, [C.c_void_p, C.c_int, C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint64, C.c_uint64]),
    "aionhip_weight_upload": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p, C.POINTER(C.c_void_p)]),
    "aionhip_weight_from_device": (C.c_int, [C.c_void_p, C.c_int, C.c_int, C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint64, C.POINTER(C.c_void_p)]),
    "aionhip_weight_free": (None, [C.c_void_p, C.c_void_p]),
    "aionhip_weight_drop_bf16": (None, [C.c_void_p, C.c_void_p]),
    "aionhip_set_bf16_weight_copies": (C.c_int, [C.c_void_p, C.c_int]),
    "aionhip_bf16_copy_stats": (C.c_int, [C.c_void_p, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "aionhip_weight_packed_bytes": (C.c_size_t, [C.c_void_p]),
    "aionhip_weight_device_bytes": (C.c_size_t, [C.c_void_p]),
    "aionhip_weight_download": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "aionhip_step_matmul": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint64, C.c_size_t, C.c_uint64, C.c_size_t, C.c_float, C.c_float]),
    "aionhip_step_matmul_nt": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint64, C.c_size_t, C.c_uint64, C.c_size_t, C.c_float, C.c_float]),
    "aionhip_step_matmul_static": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint64, C.c_size_t, C.c_uint64, C.c_size_t, C.c_float, C.c_float]),
    "aionhip_step_matmul_batch": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_void_p), C.c_size_t, C.c_uint64, C.c_size_t, C.POINTER(C.c_uint64), C.POINTER(C.c_size_t), C.c_float, C.c_float]),
    "aionhip_step_rmsnorm_matmul": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_void_p), C.c_size_t, C.c_uint64, C.c_uint64, C.c_uint64, C.c_float, C.POINTER(C.c_uint64), C.POINTER(C.c_size_t), C.c_float, C.c_float]),
    "aionhip_step_rmsnorm_qkv_rope_append": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_float,
                                                       C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_size_t, C.c_size_t, C.c_size_t,
                                                       C.c_size_t, C.c_float, C.c_float, C.c_float, C.c_int]),
    "aionhip_step_rmsnorm_geglu_matmul": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_float,
                                                    C.c_uint64, C.c_float, C.c_float]),
    "aionhip_step_gate_matmul": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint64, C.c_uint64, C.c_uint64, C.c_size_t, C.c_float, C.c_float]),
    "aionhip_step_rope_append": (C.c_int, [C.c_void_p] + [C.c_uint64] * 8 + [C.c_size_t] * 6 + [C.c_float] * 3),
    "aionhip_step_add_i32": (C.c_int, [C.c_void_p] + [C.c_uint64] * 3 + [C.c_size_t]),
    "aionhip_step_advance_state": (C.c_int, [C.c_void_p, C.c_uint64, C.c_uint64, C.c_size_t, C.POINTER(C.c_uint64), C.c_size_t, C.c_int]),
    "aionhip_step_advance_state_log": (C.c_int, [C.c_void_p, C.c_uint64, C.c_uint64, C.c_size_t, C.POINTER(C.c_uint64), C.c_size_t, C.c_int,
                                                 C.c_uint64, C.c_uint64, C.c_size_t]),
    "aionhip_decoder_stack_create": (C.c_int, [C.c_void_p, C.POINTER(DecoderStackDesc), C.POINTER(DecoderStackLayer), C.POINTER(C.c_void_p)]),
    "aionhip_decoder_stack_destroy": (None, [C.c_void_p, C.c_void_p]),
    "aionhip_step_decoder_stack": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64]),
    "aionhip_decoder_stack_status": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(C.c_int)]),
    "aionhip_decoder_stack_set_poll_budget": (C.c_int, [C.c_void_p, C.c_void_p, C.c_double]),
    "aionhip_decoder_stack_set_stamps": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint64]),
    "aionhip_program_begin": (C.c_int, [C.c_void_p]),
    "aionhip_program_end": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p)]),
    "aionhip_program_abort": (C.c_int, [C.c_void_p]),
    "aionhip_program_execute": (C.c_int, [C.c_void_p, C.c_void_p]),
    "aionhip_program_node_count": (C.c_size_t, [C.c_void_p]),
    "aionhip_program_is_current": (C.c_int, [C.c_void_p, C.c_void_p]),
    "aionhip_program_destroy": (None, [C.c_void_p, C.c_void_p]),
    "aionhip_session_create": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p)]),
    "aionhip_session_set_fusion": (C.c_int, [C.c_void_p, C.c_int]),
    "aionhip_session_execute": (C.c_int, [C.c_void_p, C.POINTER(Step), C.c_size_t]),
    "aionhip_session_stats": (C.c_int, [C.c_void_p, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "aionhip_session_retire": (C.c_int, [C.c_void_p]),
    "aionhip_session_destroy": (None, [C.c_void_p]),
    "aionhip_set_attention_precise": (C.c_int, [C.c_void_p, C.c_int]),
    "aionhip_set_gemm_mode": (C.c_int, [C.c_void_p, C.c_int]),
    "aionhip_step_attention": (C.c_int, [C.c_void_p, C.POINTER(Attention)]),
    "aionhip_step_rmsnorm": (C.c_int, [C.c_void_p] + [C.c_uint64] * 5 + [C.c_size_t, C.c_size_t, C.c_float]),
    "aionhip_step_rope": (C.c_int, [C.c_void_p] + [C.c_uint64] * 3 + [C.c_size_t] * 4 + [C.c_float] * 3),
    "aionhip_step_add": (C.c_int, [C.c_void_p] + [C.c_uint64] * 3 + [C.c_size_t]),
    "aionhip_step_gate_gelu": (C.c_int, [C.c_void_p] + [C.c_uint64] * 3 + [C.c_size_t]),
    "aionhip_step_gather_rows": (C.c_int, [C.c_void_p, C.c_int] + [C.c_uint64] * 3 + [C.c_size_t] * 3),
    "aionhip_step_append_f16": (C.c_int, [C.c_void_p] + [C.c_uint64] * 3 + [C.c_size_t] * 4 + [C.c_int]),
    "aionhip_step_sequence_append": (C.c_int, [C.c_void_p, C.c_int] + [C.c_uint64] * 3 + [C.c_size_t] * 4 + [C.c_int]),
    "aionhip_step_cast_f32_f16": (C.c_int, [C.c_void_p, C.c_uint64, C.c_uint64, C.c_size_t]),
    "aionhip_step_headnorm_rope_append": (C.c_int, [C.c_void_p] + [C.c_uint64] * 10 + [C.c_float] + [C.c_uint64] * 4 + [C.c_size_t] * 6 +
                                          [C.c_float] * 3 + [C.c_int]),
    "aionhip_step_unary": (C.c_int, [C.c_void_p, C.c_int, C.c_uint64, C.c_uint64, C.c_size_t]),
    "aionhip_step_binary": (C.c_int, [C.c_void_p, C.c_int, C.c_uint64, C.c_uint64, C.c_uint64, C.c_size_t, C.c_size_t]),
    "aionhip_cache_grow": (C.c_int, [C.c_void_p, C.c_uint64, C.c_uint64] + [C.c_size_t] * 3),
    "aionhip_cache_grow_rolling": (C.c_int, [C.c_void_p] + [C.c_uint64] * 3 + [C.c_size_t] * 5),
    "aionhip_cache_grow_target": (C.c_size_t, [C.c_size_t] * 3),
    "aionhip_probe_stream_read": (C.c_int, [C.c_void_p, C.c_uint64, C.c_size_t, C.c_size_t, C.c_uint64]),
    "aionhip_step_argmax": (C.c_int, [C.c_void_p, C.c_uint64, C.c_uint64, C.c_size_t, C.c_size_t]),
    "aionhip_event_create": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p)]),
    "aionhip_event_record": (C.c_int, [C.c_void_p, C.c_void_p]),
    "aionhip_event_elapsed_ms": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]),
    "aionhip_event_destroy": (None, [C.c_void_p, C.c_void_p]),
    "aionhip_profile_start": (C.c_int, [C.c_void_p]),
    "aionhip_profile_stop": (C.c_int, [C.c_void_p, C.POINTER(C.c_size_t)]),
    "aionhip_profile_entry": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_char_p), C.POINTER(C.c_float)]),
}

_lib = None


def load_library():
    """Loads libaion_hip.so and types every entry point. Raises if the library is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError(
            "%s is missing: build it with `python -m aion_amd.build` (there is no CPU fallback)" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in _SIGS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib
