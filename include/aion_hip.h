/* aion_hip.h - C ABI of the MI355X (gfx950) execution backend for aion's quantized-inference
 * hot path: q4_0/q8_0 dequant-fused GEMV (decode), q4/q8 GEMM (prefill), fused causal/GQA
 * attention over a KV cache, plus the small per-token ops a decoder needs between them.
 *
 * The library (libaion_hip.so) is what an aion `Backend`/`Session`/`DeviceMemory` implementation
 * written in Zig binds through @cImport: plain pointers, sizes and enums only. Citations name
 * the aion interface each entry point stands in for (paths relative to the aion source tree).
 *
 * Conventions
 *  - Every function returning `int` returns an aionhip_status. On failure a message is kept
 *    per context (aionhip_last_error).
 *  - aionhip_handle is a device address as u64 (aion `DeviceHandle`, runtime/device_memory.zig:
 *    0 = none). Step functions take device addresses; offsets are applied by the caller.
 *  - All launches are asynchronous on the context's one HIP stream. aionhip_d2h and
 *    aionhip_sync are the synchronisation points (backend/gpu/backend.zig:178-183). A context
 *    is not thread-safe; use one per session thread.
 *  - Index operands (positions, kv lengths, write index, token ids) are read ON DEVICE
 *    (backend/gpu/exec/decode_ops.zig:441-480): no step synchronises with the host.
 */
#ifndef AION_HIP_H
#define AION_HIP_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* BackendError + StoreError (backend/types.zig:27, runtime/tensor_store.zig:7), numbered like
 * AionStatus (include/aion.h:62-68). */
typedef enum aionhip_status {
    AIONHIP_OK = 0,
    AIONHIP_INVALID_ARGUMENT = 1,
    AIONHIP_OUT_OF_MEMORY = 2,
    AIONHIP_UNSUPPORTED = 3,
    AIONHIP_EXECUTION_FAILED = 4,
} aionhip_status;

/* DType ids (backend/types.zig:29-39, include/aion.h:70-77). BF16 is a host-view element type
 * in aion (include/aion.h:171-176); here it is also accepted for attention operands. */
typedef enum aionhip_dtype {
    AIONHIP_F32 = 0,
    AIONHIP_F16 = 1,
    AIONHIP_I8 = 2,
    AIONHIP_Q4_0 = 3,
    AIONHIP_Q8_0 = 4,
    AIONHIP_I32 = 5,
    AIONHIP_BF16 = 16,
} aionhip_dtype;

/* Where the 32-element quant blocks of a rank-2 weight run (storage/quantize.zig:31-80):
 * ROWS_NK = B stored [N,K], quant_axis 1 (the MatMulNT operand, runtime/executable.zig:211-223);
 * KMAJOR_KN = B stored [K,N], quant_axis 0 (the MatMul operand; the only q4_0 layout,
 * cpu/exec/matmul.zig:233-239,436-443). */
typedef enum aionhip_weight_layout {
    AIONHIP_ROWS_NK = 0,
    AIONHIP_KMAJOR_KN = 1,
} aionhip_weight_layout;

typedef struct aionhip_ctx aionhip_ctx;
typedef struct aionhip_weight aionhip_weight;
typedef struct aionhip_program aionhip_program;
typedef uint64_t aionhip_handle;

/* ---- backend handle: Backend.VTable / Session.VTable (backend/backend.zig:24-107) ---------- */
/* `stream`: a hipStream_t to launch on, or NULL to create a private stream. */
int aionhip_create(int device, void *stream, aionhip_ctx **out);
void aionhip_destroy(aionhip_ctx *ctx);                 /* Backend.deinit */
int aionhip_sync(aionhip_ctx *ctx);                     /* Session.retireResources: wait for the stream */
const char *aionhip_last_error(aionhip_ctx *ctx);       /* diagnostic.zig:1-45 analogue */
const char *aionhip_name(void);                         /* Backend.name */
void *aionhip_stream(aionhip_ctx *ctx);                 /* the hipStream_t steps launch on */
/* device facts for roofline reports: compute units, wavefront size, HBM bytes */
int aionhip_device_info(aionhip_ctx *ctx, int *cu_count, int *wave_size, uint64_t *hbm_bytes, char *arch, size_t arch_len);

/* ---- DeviceMemory.VTable (runtime/device_memory.zig:36-108); memory model = discrete,
 *      maxBindingBytes = unbounded (tensors are never chunked, storage/layout.zig:22-39) ------ */
/* alloc / free go through a pool kept by the context: a freed block of up to 64 MiB stays with the context under its size
 * class (at most 12.5 % above the request) and serves the next request of that class, in stream order, without the
 * device-wide wait of a hipFree (aion's WebGPU backend keeps grow-only pooled device buffers the same way,
 * backend/gpu/context.zig:80-110; its activations live in planned workspace slots, graph/program/workspace.zig:1-60).
 * An allocation that fails for lack of memory releases the cached blocks and is tried once more. */
int aionhip_alloc(aionhip_ctx *ctx, size_t bytes, size_t alignment, aionhip_handle *out);
void aionhip_free(aionhip_ctx *ctx, aionhip_handle h);
/* gives the cached blocks back to the device (waits for the stream); bytes handed out / bytes cached by the pool */
int aionhip_trim(aionhip_ctx *ctx);
int aionhip_memory_stats(aionhip_ctx *ctx, uint64_t *live_bytes, uint64_t *cached_bytes);
int aionhip_h2d(aionhip_ctx *ctx, aionhip_handle dst, size_t dst_offset, const void *src, size_t bytes);
int aionhip_d2h(aionhip_ctx *ctx, void *dst, aionhip_handle src, size_t src_offset, size_t bytes);
int aionhip_d2d(aionhip_ctx *ctx, aionhip_handle dst, size_t dst_offset, aionhip_handle src, size_t src_offset, size_t bytes);
int aionhip_memset(aionhip_ctx *ctx, aionhip_handle dst, size_t dst_offset, int value, size_t bytes);

/* ---- quantizers ----------------------------------------------------------------------------
 * Host: storage/quantize.zig:31-80 `quantizeBlocks` (same argument meaning: blocks
 * [first_block, first_block + out_len/block_bytes) of a tensor of `shape`, `values` holding the
 * row-major elements from `first_elem` on). q8_0 follows packQ8Block (:83-103); q4_0 follows
 * quantizeQ4_0FromF32Block32 (cpu/test_cpu_kernels.zig:490-523), the only q4 quantizer aion has. */
int aionhip_quantize_blocks(int dtype, const size_t *shape, size_t rank, size_t quant_axis,
                            const float *values, size_t n_values, size_t first_elem, size_t first_block,
                            uint8_t *out, size_t out_len);
/* Device: the same bytes for a rank-2 f32 tensor `src` [rows, cols] resident on the GPU
 * (Context.quantize, api/context.zig:443-489, without the host round trip). */
int aionhip_quantize_device(aionhip_ctx *ctx, int dtype, size_t rows, size_t cols, size_t quant_axis,
                            aionhip_handle src_f32, aionhip_handle dst_blocks);

/* ---- weights: private re-lay at first use (graph/opt/weight_layout.zig:232-314 does the same
 *      job for the CPU/WebGPU block orders; this backend advertises `.row_major`,
 *      api/gpu_device.zig:24-25, and keeps its own layout) -----------------------------------
 * Input is aion's packed blocks, exactly as the quantizer emits them: ROWS_NK -> block (n,kb)
 * at (n*K/32+kb)*block_bytes; KMAJOR_KN -> block (kb,n) at (kb*ld+n)*block_bytes (ld = row
 * stride in blocks, 0 = n; MatMulParams.ldb, backend/types.zig:225-241). Of the block formats only Q8_0 may be
 * ROWS_NK. dtype AIONHIP_F32 with ROWS_NK is the f32 operand of MatMulNT (runtime/executable.zig:211-223,
 * cpu/exec/matmul_nt.zig:100): n rows of k floats, kept as they are (any k, ld_blocks 0); such a weight is accepted by
 * aionhip_step_matmul_nt only - the batched and fused steps answer AIONHIP_UNSUPPORTED and the caller issues the separate
 * steps. The bytes handed in are consumed during the call and not referenced afterwards. */
int aionhip_weight_upload(aionhip_ctx *ctx, int dtype, int layout, size_t n, size_t k, size_t ld_blocks,
                          const void *host_blocks, aionhip_weight **out);
/* same, from blocks already resident in device memory (a tensor moved by DeviceMemory.copyH2D) */
int aionhip_weight_from_device(aionhip_ctx *ctx, int dtype, int layout, size_t n, size_t k, size_t ld_blocks,
                               aionhip_handle device_blocks, aionhip_weight **out);
void aionhip_weight_free(aionhip_ctx *ctx, aionhip_weight *w);
/* bytes of aion's packed form (what the roofline charges) and of the device layout */
size_t aionhip_weight_packed_bytes(const aionhip_weight *w);
size_t aionhip_weight_device_bytes(const aionhip_weight *w);
/* Inverse of the re-lay: aion's packed blocks back out of the device layout (byte-exact) */
int aionhip_weight_download(aionhip_ctx *ctx, const aionhip_weight *w, void *host_blocks, size_t bytes);

/* ---- matmul steps -----------------------------------------------------------------------------
 * StepMatMul (B [K,N], cpu/exec/matmul.zig:48-78) and StepMatMulNT (B [N,K],
 * cpu/exec/matmul_nt.zig:87-259): C[m,n] = alpha * A[m,k] @ B + beta * C, A and C f32 on device,
 * lda/ldc in elements (0 = k / n). Leading dims of A are folded into m by the caller
 * (cpu/exec/matmul.zig:100-163). Arithmetic follows aion's CPU kernels: A is int8-quantized
 * per (row, 32-block) (cpu/kernels/matmul_q_i8.zig:187-203), block dots are exact integers,
 * accumulation is f32. MatMulNT with an f32 weight (cpu/kernels/matmul_nt.zig:40-126) quantizes nothing: f32 fused
 * multiply-adds over k, f32 sums. */
int aionhip_step_matmul(aionhip_ctx *ctx, const aionhip_weight *b, size_t m,
                        aionhip_handle a, size_t lda, aionhip_handle c, size_t ldc, float alpha, float beta);
int aionhip_step_matmul_nt(aionhip_ctx *ctx, const aionhip_weight *b, size_t m,
                           aionhip_handle a, size_t lda, aionhip_handle c, size_t ldc, float alpha, float beta);

/* aionhip_step_matmul / aionhip_step_matmul_nt (by the weight's layout) for callers that cannot allocate: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc. No counterpart in aion. Same kernels and the
 * same results as the two entry points above, but the prepared activation (int8 codes, block scales, block code
 * sums: m * k + m * k / 32 * 8 bytes, each plane rounded up to 256) lives in a file-scope device array of
 * AIONHIP_STATIC_SCRATCH_BYTES instead of the context's growable scratch, and the call makes no hipMalloc / hipFree or
 * other allocating call. AIONHIP_INVALID_ARGUMENT when the prepared activation of (m, k) does not fit the array;
 * AIONHIP_UNSUPPORTED for m > 8 under a bf16 GEMM mode (that path builds weight copies) and while per-launch
 * profiling is on (it creates events). Each GPU holds one array, shared by every context on it and keeping the last
 * call's contents: calls that overlap on one GPU (two contexts, two streams) race. */
#define AIONHIP_STATIC_SCRATCH_BYTES ((size_t)1 << 20)
int aionhip_step_matmul_static(aionhip_ctx *ctx, const aionhip_weight *b, size_t m,
                               aionhip_handle a, size_t lda, aionhip_handle c, size_t ldc, float alpha, float beta);

/* Several matmul steps that read the SAME activation (q/k/v, gate/up) as one call: the activation
 * is prepared once and, for m <= 8, all weights stream through one launch. aion keeps such
 * siblings as separate MatMul/MatMulNT steps (graph/opt/weight_layout.zig:72-115 re-lays but never
 * concatenates); every C[i] is what the separate step would have produced. count <= 4; weights
 * share k and dtype; ldc may be NULL (each n). */
int aionhip_step_matmul_batch(aionhip_ctx *ctx, size_t count, const aionhip_weight *const *b, size_t m,
                              aionhip_handle a, size_t lda, const aionhip_handle *c, const size_t *ldc,
                              float alpha, float beta);

/* Decode fusion of one attention block's input side for ONE new token of ONE sequence: RMSNorm(x) -> the
 * q, k and v matmuls (StepMatMul x3 on the same activation) -> RoPE on q and k (StepRope, chunked halves,
 * cpu/kernels/rope.zig:20-98) -> f32->f16 cast and append of k and v at the device-resident write index
 * (StepSequenceAppend, cpu/exec/sequence_append.zig:12-104), as one launch. q_out receives the rotated
 * query [h_q, d] f32; the caches are [t_cap, h_kv, d] f16 (batch 1). Same arithmetic as the separate steps
 * (aionhip_step_rmsnorm_matmul + aionhip_step_rope_append); rolling = 1: the caches are rings, as in
 * aionhip_step_append_f16. AIONHIP_UNSUPPORTED when the shape does not qualify (k above 8192, misaligned
 * operands): the caller then issues the separate steps. */
int aionhip_step_rmsnorm_qkv_rope_append(aionhip_ctx *ctx, const aionhip_weight *wq, const aionhip_weight *wk, const aionhip_weight *wv,
                                         aionhip_handle x, aionhip_handle gamma, aionhip_handle beta_norm, float eps,
                                         aionhip_handle q_out, aionhip_handle k_cache, aionhip_handle v_cache,
                                         aionhip_handle positions, aionhip_handle write_index, size_t t_cap, size_t h_q, size_t h_kv,
                                         size_t d, float base_frequency, float scale_factor, float rope_proportion, int rolling);
/* Decode fusion of a GeGLU feed-forward block for ONE activation row: RMSNorm(x) -> gate and up matmuls ->
 * gate(gelu_tanh) * up (cpu/exec/elementwise.zig:25-37) -> int8 activation preparation -> down matmul,
 * C[1, n_down] = alpha * (...) + beta * C, in two launches; the gate / up / gated rows never reach memory.
 * Same arithmetic as aionhip_step_rmsnorm_matmul + aionhip_step_gate_matmul. AIONHIP_UNSUPPORTED when the
 * shape does not qualify (k above 8192, hidden size not a multiple of 32, misaligned operands). */
int aionhip_step_rmsnorm_geglu_matmul(aionhip_ctx *ctx, const aionhip_weight *w_gate, const aionhip_weight *w_up, const aionhip_weight *w_down,
                                      aionhip_handle x, aionhip_handle gamma, aionhip_handle beta_norm, float eps,
                                      aionhip_handle c, float alpha, float beta);
/* StepRMSNorm feeding MatMul steps, and the fused gate feeding a MatMul step, as one call each:
 * the normalised (or gated) activation is not written out; for one row it is built inside the GEMV
 * kernel, for more rows on the exact kernels the norm (or gate) and the int8 preparation are one launch. Same arithmetic as aionhip_step_rmsnorm / aionhip_step_gate_gelu followed by the matmul
 * step(s). aion fuses at step level the same way (RMSNorm.residual, ElemwiseBinary.gate:
 * graph/opt/fuse_steps.zig:19-88); these two go one step further because a decode step on this
 * GPU is bound by launch count, not bandwidth. */
int aionhip_step_rmsnorm_matmul(aionhip_ctx *ctx, size_t count, const aionhip_weight *const *b, size_t rows,
                                aionhip_handle x, aionhip_handle gamma, aionhip_handle beta_norm, float eps,
                                const aionhip_handle *c, const size_t *ldc, float alpha, float beta);
int aionhip_step_gate_matmul(aionhip_ctx *ctx, const aionhip_weight *b, size_t rows, aionhip_handle gate, aionhip_handle up,
                             aionhip_handle c, size_t ldc, float alpha, float beta);

/* How m > 8 rows are multiplied. EXACT_I8 (default): int8 activations, integer MFMA, per-block
 * f32 scaling - the same numbers as the decode path. BF16_MFMA: weights dequantized to bf16 (a copy the context
 * keeps, or while the kernel stages them: aionhip_set_bf16_weight_copies), activations rounded to bf16, f32
 * accumulation - judged at 1e-2 instead of 2e-3; used where it is expected to
 * be the faster kernel (from a few hundred rows on; below that the exact kernel runs, which is then both faster
 * and exact). BF16_MFMA_ALWAYS: the bf16 kernel for every m > 8, whatever the shape. */
typedef enum aionhip_gemm_mode { AIONHIP_GEMM_EXACT_I8 = 0, AIONHIP_GEMM_BF16_MFMA = 1, AIONHIP_GEMM_BF16_MFMA_ALWAYS = 2 } aionhip_gemm_mode;
int aionhip_set_gemm_mode(aionhip_ctx *ctx, int mode);
/* The weight operand of the bf16 kernel. on (default): the context keeps a bf16 copy of every weight it has multiplied in
 * bf16 mode (n rounded up to 16, times k * 2 bytes - about four times a q4_0 weight), built on the weight's first such call,
 * never while a program is being recorded, owned by the context (no other context sees it) and released by
 * aionhip_weight_drop_bf16, aionhip_weight_free through the same context, or aionhip_destroy; aion's derived weights
 * (storage/derived.zig:1-17) are the counterpart. off: no copies - the kernel converts the quant blocks while it stages
 * them, as aion's GPU GEMM does (backend/gpu/kernels/matmul_q8_mx16.wgsl); nothing resident and nothing allocated, at
 * about three quarters of the speed (measured: 264 against 197 us for 2048 x 14336 x 4096). Same results to the bit. */
int aionhip_set_bf16_weight_copies(aionhip_ctx *ctx, int on);
void aionhip_weight_drop_bf16(aionhip_ctx *ctx, aionhip_weight *w);       /* waits for the context's stream */
int aionhip_bf16_copy_stats(aionhip_ctx *ctx, uint64_t *weights, uint64_t *bytes);
/* Name of the kernel the last matmul/attention step launched (the reference's tests assert
 * which kernel ran after a parity check, backend/gpu/test_gpu_backend.zig:1116-1162). */
const char *aionhip_last_kernel(aionhip_ctx *ctx);
/* The last launch a matmul or fused step made, for reports that are matched against a kernel trace: the kernel instance's
 * name as a trace prints it (demangled, template arguments included, no parameter list), its grid in workgroups, its
 * workgroup size and its dynamic LDS bytes. Any pointer may be NULL. aion's counterpart is the WebGPU backend's per-dispatch
 * labels (backend/gpu/timestamp_profile.zig). */
int aionhip_last_launch(aionhip_ctx *ctx, char *instance, size_t instance_len, unsigned grid[3], unsigned block[3], size_t *lds_bytes);

/* ---- attention step: StepAttention (runtime/executable.zig:102-115), graph.Op.Attention
 *      (graph/graph.zig:365-393), executor cpu/exec/attention.zig:1444-1608 ------------------
 * q [B,L,Hq,Dk], k [B,T,Hkv,Dk], v [B,T,Hkv,Dv] token-major, out f32 [B,L,Hq,Dv]. Key interval
 * per query = AttentionWindow.keys(pos, end) (graph/graph.zig:160-167); 0xFFFFFFFF = unbounded,
 * causal = {left unbounded, right 0, chunk 0}. query_positions [B,L] i32 / kv_lengths [B] i32
 * are device addresses or 0 (defaults: row index / T). Empty interval -> zeros. */
typedef struct aionhip_attention {
    aionhip_handle out, q, k, v, query_positions, kv_lengths;
    size_t batch, l_q, t_kv, h_q, h_kv, d_k, d_v;
    int q_dtype;   /* F32 | F16 | BF16 */
    int kv_dtype;  /* F32 | F16 | BF16 */
    float scale, attn_logits_soft_cap;
    uint32_t window_left, window_right, window_chunk;
    /* 1: k and v are rolling caches (storage/cache.zig:35-38, 202-207): logical key t lives in row t % T,
     * kv_lengths may exceed T, and keys older than kv_length - T are gone (cpu/exec/attention.zig:1072-1075,
     * 1150-1152, 1537-1546). 0: row t is key t and kv_lengths is clipped to T. */
    uint32_t rolling;
} aionhip_attention;
int aionhip_step_attention(aionhip_ctx *ctx, const aionhip_attention *p);
/* f32 queries over an f16/bf16 cache: off (default) = q rounded to the cache element type, one MFMA
 * pass (2e-3 tolerance class); on = q and the probabilities fed as hi+lo parts (agrees with an f64
 * reference to ~1e-6, about 1.4x the kernel time at decode). */
int aionhip_set_attention_precise(aionhip_ctx *ctx, int on);

/* ---- per-token glue steps (f32 unless stated) ---------------------------------------------- */
/* StepRMSNorm (runtime/executable.zig:85-101; cpu/exec/layernorm.zig:54-155):
 * out = x * rsqrt(mean(x^2)+eps) * gamma + beta (+ residual). beta/residual may be 0. */
int aionhip_step_rmsnorm(aionhip_ctx *ctx, aionhip_handle out, aionhip_handle x, aionhip_handle gamma,
                         aionhip_handle beta, aionhip_handle residual, size_t rows, size_t cols, float eps);
/* StepRoPE1D (cpu/exec/rope.zig:14-53, cpu/kernels/rope.zig:20-98): x,out [B,T,H,D], positions [B,T] i32 */
int aionhip_step_rope(aionhip_ctx *ctx, aionhip_handle out, aionhip_handle x, aionhip_handle positions,
                      size_t b, size_t t, size_t h, size_t d, float base_frequency, float scale_factor, float rope_proportion);
/* RoPE1D(q) + RoPE1D(k) + Cast f16 + SequenceAppend(k cache) + Cast f16 + SequenceAppend(v cache)
 * of one step as a single launch (same arithmetic as the separate steps): q,q_out [B,S,Hq,D] f32,
 * k,v [B,S,Hkv,D] f32, caches [B,T,Hkv,D] f16, positions [B,S] i32, write_index [B] i32 on device */
int aionhip_step_rope_append(aionhip_ctx *ctx, aionhip_handle q_out, aionhip_handle q, aionhip_handle k, aionhip_handle v,
                             aionhip_handle k_cache, aionhip_handle v_cache, aionhip_handle positions, aionhip_handle write_index,
                             size_t b, size_t s, size_t t_cap, size_t h_q, size_t h_kv, size_t d,
                             float base_frequency, float scale_factor, float rope_proportion);
/* The same with an RMSNorm over the head dimension on q, k and v in front (StepRMSNorm x3, gamma / beta of width d,
 * a beta may be 0; cpu/exec/layernorm.zig:54-155): the input side of an attention block in models that normalize
 * their heads (src/bench/models.zig:455-473), one launch instead of eight to ten. rope_proportion 0 = no rotation;
 * rolling = 1: ring caches. Head sizes up to 512 (AIONHIP_UNSUPPORTED above: issue the separate steps). */
int aionhip_step_headnorm_rope_append(aionhip_ctx *ctx, aionhip_handle q_out, aionhip_handle q, aionhip_handle k, aionhip_handle v,
                                      aionhip_handle gamma_q, aionhip_handle beta_q, aionhip_handle gamma_k, aionhip_handle beta_k,
                                      aionhip_handle gamma_v, aionhip_handle beta_v, float eps, aionhip_handle k_cache,
                                      aionhip_handle v_cache, aionhip_handle positions, aionhip_handle write_index, size_t b, size_t s,
                                      size_t t_cap, size_t h_q, size_t h_kv, size_t d, float base_frequency, float scale_factor,
                                      float rope_proportion, int rolling);
/* StepElemwiseBinary: add, and the fused gate act(a)*b with act = gelu (tanh form)
 * (backend/types.zig:105-109, cpu/exec/elementwise.zig:25-37, cpu/kernels/gelu.zig:8-14) */
int aionhip_step_add(aionhip_ctx *ctx, aionhip_handle out, aionhip_handle a, aionhip_handle b, size_t n);
int aionhip_step_gate_gelu(aionhip_ctx *ctx, aionhip_handle out, aionhip_handle a, aionhip_handle b, size_t n);
/* StepUnary on f32 (backend/types.zig:119-128 UnaryOp, the ids below are its ids; cpu/exec/unary.zig:55-64):
 * sigmoid and tanh are aion's exp-based approximations (cpu/kernels/fast_math.zig:53-148), gelu the tanh form
 * (cpu/kernels/gelu.zig:8-14), silu = x * sigmoid(x). log (id 6): AIONHIP_UNSUPPORTED. out may alias x. */
enum { AIONHIP_UNARY_RELU = 0, AIONHIP_UNARY_GELU = 1, AIONHIP_UNARY_SILU = 2, AIONHIP_UNARY_SIGMOID = 3,
       AIONHIP_UNARY_TANH = 4, AIONHIP_UNARY_SQRT = 5 };
int aionhip_step_unary(aionhip_ctx *ctx, int op, aionhip_handle out, aionhip_handle x, size_t n);
/* StepElemwiseBinary add / sub / mul / div on f32 (backend/types.zig:92-96 ElemwiseBinaryOp ids;
 * cpu/exec/elementwise.zig:38-60): b has a's n elements (identical), one element (scalar_b) or the nb elements of
 * a contiguous suffix of a's shape (contiguous_suffix_b): out[i] = a[i] op b[i % nb]. The comparison ops and general
 * broadcasts: AIONHIP_UNSUPPORTED. out may alias a. */
enum { AIONHIP_BINARY_ADD = 0, AIONHIP_BINARY_SUB = 1, AIONHIP_BINARY_MUL = 2, AIONHIP_BINARY_DIV = 3 };
int aionhip_step_binary(aionhip_ctx *ctx, int op, aionhip_handle out, aionhip_handle a, aionhip_handle b, size_t n, size_t nb);
/* StepGather axis 0 (cpu/exec/gather.zig:60-87): rows of an f32 or q8_0 (quant_axis 1, packed
 * 34-byte blocks) table [V,D] -> out f32 [n_ids, D]; ids i32 on device */
int aionhip_step_gather_rows(aionhip_ctx *ctx, int table_dtype, aionhip_handle out, aionhip_handle table,
                             aionhip_handle ids, size_t n_ids, size_t d, size_t vocab);
/* StepCast f32 -> f16 (cpu/exec/cast.zig) fused with StepSequenceAppend
 * (cpu/exec/sequence_append.zig:12-104): rows src [B,S,H,D] f32 are written as f16 into
 * cache [B,T,H,D] at token index write_index[b] (i32 [B] on device) .. +S; rolling = 1: the cache is a ring
 * and logical step t goes to row t % T (storage/cache.zig:202-207) */
int aionhip_step_append_f16(aionhip_ctx *ctx, aionhip_handle cache, aionhip_handle src_f32, aionhip_handle write_index,
                            size_t b, size_t s, size_t t_cap, size_t row_elems, int rolling);
int aionhip_step_cast_f32_f16(aionhip_ctx *ctx, aionhip_handle out_f16, aionhip_handle x_f32, size_t n);
/* StepSequenceAppend as the step itself (runtime/executable.zig:193-206, cpu/exec/sequence_append.zig:12-104): cache
 * [B,T,H,D] and new_kv [B,S,H,D] of the same element type `dtype` (AIONHIP_F16 or AIONHIP_F32), end_index i32 [B] on the
 * device; rows go to token index end_index[b] .. +S (rolling = 1: to row t % T). A row that would fall outside a linear
 * cache is not written (the reference rejects the step on the host before any write; capacity is settled before the
 * program runs, api/loaded_model.zig:791-827). */
int aionhip_step_sequence_append(aionhip_ctx *ctx, int dtype, aionhip_handle cache, aionhip_handle new_kv, aionhip_handle end_index,
                                 size_t b, size_t s, size_t t_cap, size_t row_elems, int rolling);
/* Growth of a sequence cache along its time axis with the data kept on the device
 * (storage/manager/grow.zig:37-78 growAxisOnDevice, driven by api/loaded_model.zig:791-827 and
 * storage/manager/store_view.zig:104-124): dst is the new backing [outer, new_run_bytes], src the old one
 * [outer, old_run_bytes]; every run is copied to the start of its wider slot and the rest of dst is zero. Runs are
 * whole 4-byte words (grow.zig:51-52) and new_run_bytes >= old_run_bytes. For a cache [B,T,H,D] grown to T':
 * outer = B, runs = T*H*D and T'*H*D elements. dst and src are distinct buffers; the caller frees src afterwards
 * (stream order keeps it alive for this copy). */
int aionhip_cache_grow(aionhip_ctx *ctx, aionhip_handle dst, aionhip_handle src, size_t outer, size_t old_run_bytes,
                       size_t new_run_bytes);
/* The same for a rolling cache [B, capacity, row] (grow.zig:107-150 ensureRollingCacheCapacity, which goes through the
 * host; here one kernel): the row of logical step t is t % capacity, so the retained steps of batch entry b - the last
 * min(end, retained_history, old_capacity) steps before end = logical_ends[b] (i32 [B] on device) - move to row
 * t % new_capacity; all other rows of dst are zero. new_capacity > old_capacity > 0. */
int aionhip_cache_grow_rolling(aionhip_ctx *ctx, aionhip_handle dst, aionhip_handle src, aionhip_handle logical_ends, size_t b,
                               size_t old_capacity, size_t new_capacity, size_t row_bytes, size_t retained_history);
/* The next capacity of a geometric growth schedule (storage/manager.zig:69-76 growTarget, storage/cache.zig:129-137):
 * ceil(current * num / den), or current + 1 where that is no growth. 0 = invalid argument or overflow. Host only. */
size_t aionhip_cache_grow_target(size_t current, size_t num, size_t den);
/* Measurement aid with no counterpart in aion: reads `bytes` of `src` from byte `offset` with a plain
 * streaming kernel and discards them (`sink`: any 4-byte device buffer, normally left untouched). Timed by
 * the profiler as "stream_read"; bench.py reports the GEMV kernels beside it. offset, bytes: multiples of 16. */
int aionhip_probe_stream_read(aionhip_ctx *ctx, aionhip_handle src, size_t offset, size_t bytes, aionhip_handle sink);
/* StepArgMax over the last axis, first maximum wins (cpu/exec/argmax.zig:56-81); out i32 [rows] */
int aionhip_step_argmax(aionhip_ctx *ctx, aionhip_handle out_i32, aionhip_handle x, size_t rows, size_t n);

/* i32 elementwise add (StepElemwiseBinary on i32, cpu/exec/elementwise.zig): advances positions,
 * the cache write index and kv lengths on the device between replays of a decode program */
int aionhip_step_add_i32(aionhip_ctx *ctx, aionhip_handle out, aionhip_handle a, aionhip_handle b, size_t n);

/* The same bookkeeping as one launch (a decode step is bound by its launch count): dst_tokens[0..n_tokens) = src_tokens[...]
 * (i32, the token the step produced becomes the next step's input; StepCopy, runtime/executable.zig) and delta is added to
 * each of up to 8 distinct scalar i32 device values (positions, write index, visible end). */
int aionhip_step_advance_state(aionhip_ctx *ctx, aionhip_handle dst_tokens, aionhip_handle src_tokens, size_t n_tokens,
                               const aionhip_handle *counters, size_t n_counters, int delta);
/* The same, and the tokens are also written to log[*log_index .. + n_tokens) (i32; *log_index is a device scalar read
 * before the counters move and may be one of them, e.g. the position; writes past log_capacity are dropped; at most 64
 * tokens per step): a device-resident greedy loop then needs no read-back per step, the host collects the tokens when it
 * wants them (aion's sessions keep the loop state on the device the same way, api/loaded_model.zig:735-827). */
int aionhip_step_advance_state_log(aionhip_ctx *ctx, aionhip_handle dst_tokens, aionhip_handle src_tokens, size_t n_tokens,
                                   const aionhip_handle *counters, size_t n_counters, int delta,
                                   aionhip_handle log, aionhip_handle log_index, size_t log_capacity);

/* ---- a whole run of decoder blocks for ONE new token of ONE sequence, as one launch ----------
 * Session.execute receives the whole ExecutableProgram (backend/backend.zig:42-44); a decoder's program repeats
 * one block per layer (src/bench/models.zig:433-536): RMSNorm -> MatMul q,k,v -> RoPE1D(q,k) -> Cast f16 +
 * SequenceAppend(k,v) -> Attention -> MatMul o, beta = 1 (residual) -> RMSNorm -> MatMul gate,up -> gate(gelu) ->
 * MatMul down, beta = 1. aionhip_step_decoder_stack runs `layers` such blocks in one cooperative launch of one
 * workgroup per CU; between the phases of a block the small activation vectors travel through device memory as
 * self-validating words, so no step boundary costs a dispatch. Same arithmetic per output as the separate steps
 * (aionhip_step_rmsnorm_qkv_rope_append, aionhip_step_attention, aionhip_step_matmul, aionhip_step_rmsnorm_geglu_matmul).
 * create returns AIONHIP_UNSUPPORTED for shapes outside its limits (head size 128 or 256, hidden and heads x head
 * size up to 8192, ffn up to 32768, linear f16 caches, one block format for all weights): the caller then issues
 * the separate steps. Weights, gammas and caches must outlive the stack. The launch waits for nothing on the host;
 * every wait inside the kernel is bounded (250 ms by default), and aionhip_decoder_stack_status - a synchronising
 * call - returns AIONHIP_EXECUTION_FAILED if a launch since the last call ran out of that time (its outputs are
 * invalid; the stack is reset and usable again). */
typedef struct aionhip_decoder_stack aionhip_decoder_stack;
typedef struct aionhip_decoder_stack_layer {
    const aionhip_weight *wq, *wk, *wv, *wo, *w_gate, *w_up, *w_down;
    aionhip_handle norm1_gamma, norm1_beta; /* f32 [hidden]; beta 0 = none */
    aionhip_handle norm2_gamma, norm2_beta;
    aionhip_handle k_cache, v_cache;        /* f16 [t_cap, kv_heads, head_dim] */
} aionhip_decoder_stack_layer;
typedef struct aionhip_decoder_stack_desc {
    size_t layers, hidden, heads, kv_heads, head_dim, ffn, t_cap;
    float eps1, eps2;                        /* RMSNorm in front of q/k/v and in front of gate/up */
    float rope_base, rope_scale, rope_proportion;
    float attn_scale, attn_logits_soft_cap;  /* StepAttention (runtime/executable.zig:102-115) */
    uint32_t window_left, window_right, window_chunk;
    int rolling;                             /* must be 0: ring caches take the separate steps */
} aionhip_decoder_stack_desc;
int aionhip_decoder_stack_create(aionhip_ctx *ctx, const aionhip_decoder_stack_desc *desc, const aionhip_decoder_stack_layer *layers,
                                 aionhip_decoder_stack **out);
void aionhip_decoder_stack_destroy(aionhip_ctx *ctx, aionhip_decoder_stack *stack);
/* x_in, x_out: f32 [hidden] (may be the same buffer); positions [1], write_index [1], kv_lengths [1]: i32, read on the device */
int aionhip_step_decoder_stack(aionhip_ctx *ctx, aionhip_decoder_stack *stack, aionhip_handle x_in, aionhip_handle x_out,
                               aionhip_handle positions, aionhip_handle write_index, aionhip_handle kv_lengths);
int aionhip_decoder_stack_status(aionhip_ctx *ctx, aionhip_decoder_stack *stack, int *failed);
/* the time a workgroup may wait for another's results before the launch gives up (tests set it to 0 to take that path) */
int aionhip_decoder_stack_set_poll_budget(aionhip_ctx *ctx, aionhip_decoder_stack *stack, double milliseconds);
/* diagnostics: with a buffer of 2 x layers x 10 i64 (0 = off) two workgroups (the first and the middle one) note the wall
 * clock (100 MHz) when each of the five phases of every layer had its input and when its output was out */
int aionhip_decoder_stack_set_stamps(aionhip_ctx *ctx, aionhip_decoder_stack *stack, aionhip_handle stamps);

/* ---- programs: record a fixed step sequence once, replay it per token ----------------------
 * Session.execute(prog) (backend/backend.zig:42-44) runs aion's ExecutableProgram step list; the
 * WebGPU backend replays cached dispatch state because a decode program is identical every token
 * (backend/gpu/frame.zig:77-86). Between program_begin and program_end the aionhip_step_* calls
 * are recorded into a HIP graph instead of executed; program_execute replays it (asynchronous).
 * While recording: no h2d/d2h/free/sync, no profiling, and scratch cannot grow - run the same
 * steps once eagerly first. Per-token inputs must live in device buffers the steps read.
 * Lifetime: a program's launches hold the addresses of the context's work buffers (prepared
 * activations, GEMM staging, K-split words, argmax tickets). When a later eager step needs a
 * larger one (a longer prompt, more rows), the buffer is replaced and every program recorded
 * before that is stale: program_execute then returns AIONHIP_INVALID_ARGUMENT without launching
 * anything (aionhip_last_error says "stale program"), and the caller destroys it and records the
 * steps again. aionhip_program_is_current tells the same without an error. */
int aionhip_program_begin(aionhip_ctx *ctx);
int aionhip_program_end(aionhip_ctx *ctx, aionhip_program **out);
/* Leaves a recording without a program (for a caller whose step failed between begin and end): the captured work is
 * dropped and the context executes eagerly again. No-op when nothing is being recorded. */
int aionhip_program_abort(aionhip_ctx *ctx);
int aionhip_program_execute(aionhip_ctx *ctx, aionhip_program *prog);
size_t aionhip_program_node_count(const aionhip_program *prog);
/* 1 when the program may still run on this context, 0 when a work buffer it uses has been replaced since */
int aionhip_program_is_current(const aionhip_ctx *ctx, const aionhip_program *prog);
void aionhip_program_destroy(aionhip_ctx *ctx, aionhip_program *prog);

/* ---- Session.execute(prog): a step list in one call (backend/backend.zig:24-52) ---------------
 * The native twin of a Session over an ExecutableProgram's `steps` (runtime/executable.zig:302-345 Step, :378-400
 * ExecutableProgram): the binding turns every step whose placement is this device into one aionhip_step record - the
 * step's own attributes plus, for every TensorId, what the tensor store answers for it (runtime/tensor_store.zig:150-201:
 * device address, dtype, shape) - and hands the array over; the dispatch by tag, the shape arithmetic, the re-laid weight
 * cache and the launch-saving step patterns then live here instead of in every binding. `tag` is the Step union's tag in
 * declaration order. Executed tags: MatMul, MatMulNT (b = the packed weight tensor as it lies on the device), ElemwiseBinary
 * (f32 add/sub/mul/div with identical, scalar_b or contiguous_suffix_b broadcast; gate with gelu; i32 add), Unary, RMSNorm,
 * Attention, ArgMax (last axis), Copy, GatherRows, Gather (axis 0, no batch dims, rank-2 table), RoPE1D, SequenceAppend,
 * Cast (f32 -> f16), Transfer. Every other tag: AIONHIP_UNSUPPORTED before anything of the list has run (the list is checked
 * as a whole first), as the reference's compiler keeps steps a backend's capability set lacks on the CPU
 * (backend/backend.zig:85-107). */
#define AIONHIP_MAX_RANK 8
enum { AIONHIP_TENSOR_ROLLING = 1u,    /* a rolling sequence cache (storage/cache.zig:35-38) */
       AIONHIP_TENSOR_WORKSPACE = 2u   /* lives in a planned workspace slot (graph/program/workspace.zig:1-60): nothing reads
                                          its value after the last step of this list that does */ };
typedef struct aionhip_tensor_ref {
    aionhip_handle handle;             /* 0 = the step has no such operand */
    int32_t dtype;                     /* aionhip_dtype */
    uint32_t rank;
    uint32_t flags;
    uint32_t reserved;
    uint64_t shape[AIONHIP_MAX_RANK];
} aionhip_tensor_ref;
enum { AIONHIP_STEP_MATMUL = 0, AIONHIP_STEP_ELEMWISE_BINARY = 1, AIONHIP_STEP_UNARY = 2, AIONHIP_STEP_RMSNORM = 8,
       AIONHIP_STEP_ATTENTION = 9, AIONHIP_STEP_ARGMAX = 11, AIONHIP_STEP_COPY = 17, AIONHIP_STEP_GATHER_ROWS = 18,
       AIONHIP_STEP_GATHER = 19, AIONHIP_STEP_ROPE1D = 21, AIONHIP_STEP_SEQUENCE_APPEND = 22, AIONHIP_STEP_CAST = 31,
       AIONHIP_STEP_MATMUL_NT = 32, AIONHIP_STEP_TRANSFER = 33, AIONHIP_STEP_TAG_COUNT = 34 };
enum { AIONHIP_BINARY_GATE = 10 };     /* ElemwiseBinaryOp.gate (backend/types.zig:92-109; ids 4..9 are the i32 comparisons) */
/* Operands by tag (out / in[0..]):
 *   MatMul, MatMulNT     out = c; a, b                       alpha, beta
 *   ElemwiseBinary       out; a, b                           op (ElemwiseBinaryOp id), act (UnaryOp id of a gate), broadcast
 *                                                            (ElementwiseBroadcastKind id: 0 identical, 1 scalar_a, 2 scalar_b,
 *                                                            3 contiguous_suffix_a, 4 contiguous_suffix_b, 5 generic;
 *                                                            runtime/executable.zig:28-35)
 *   Unary                out; a                              op (UnaryOp id)
 *   RMSNorm              out; x, gamma, beta, residual?      eps
 *   Attention            out; q, k, v, query_positions?, kv_lengths?    scale, soft_cap, window_*
 *   ArgMax               out; a                              axis
 *   Copy                 out = dst; src
 *   GatherRows           out; table, indices
 *   Gather               out; data, indices                  axis, batch_dims
 *   RoPE1D               out; x, positions                   rope_base, rope_scale, rope_proportion
 *   SequenceAppend       out = cache; new_kv, end_index
 *   Cast                 out; x                              (the target type is out.dtype)
 *   Transfer             to_host = 1: in[0] = the device tensor, host receives; 0: out = the device tensor, host is read */
typedef struct aionhip_step {
    int32_t tag;
    int32_t op, act, broadcast;
    int32_t axis;
    uint32_t batch_dims;
    float alpha, beta;
    float eps;
    float scale, soft_cap;
    uint32_t window_left, window_right, window_chunk;
    float rope_base, rope_scale, rope_proportion;
    int32_t to_host;
    aionhip_tensor_ref out;
    aionhip_tensor_ref in[5];
    void *host;                        /* Transfer: the host bytes of the other side */
    uint64_t host_bytes;
} aionhip_step;

typedef struct aionhip_session aionhip_session;
/* Backend.createSession (backend/backend.zig:46-52). A session belongs to one context and one thread, and is destroyed before
 * its context (it frees its re-laid weights through it). */
int aionhip_session_create(aionhip_ctx *ctx, aionhip_session **out);
/* Which step patterns a session may run as one call (default: both). Results are the separate steps' to the bit either way.
 * AIONHIP_FUSE_SIBLINGS: consecutive MatMul / MatMulNT steps reading one activation share its preparation and, up to eight
 * rows, one launch (aionhip_step_matmul_batch); every tensor of the list is still written.
 * AIONHIP_FUSE_WORKSPACE: a step whose output is an AIONHIP_TENSOR_WORKSPACE tensor read only by the step(s) right behind
 * it is folded into them and that tensor is never written: RMSNorm (no residual) -> MatMul(s) (aionhip_step_rmsnorm_matmul),
 * gate(gelu) -> MatMul (aionhip_step_gate_matmul), Cast f32 -> f16 -> SequenceAppend (aionhip_step_append_f16); and for one
 * token of one sequence the two blocks of a decoder layer as one call each: RMSNorm -> q, k, v MatMuls -> RoPE1D on q and k ->
 * Cast + SequenceAppend of k and of v (ten steps, aionhip_step_rmsnorm_qkv_rope_append), RMSNorm -> gate and up MatMuls ->
 * gate(gelu) -> down MatMul (five steps, aionhip_step_rmsnorm_geglu_matmul); and for any batch and token count the cache
 * side of a block that normalizes its heads: RMSNorm over the head size on q, k, v -> RoPE1D on q and k -> Cast +
 * SequenceAppend of k and of v (nine steps, aionhip_step_headnorm_rope_append), and the same without the norms over linear
 * caches (six steps, aionhip_step_rope_append). A MatMul (beta 0) whose workspace output is
 * read only by an add right behind it that accumulates in place (x = x + t) writes x itself with beta 1, alone or as the
 * last step of the patterns above: alpha * acc + x is rounded once either way. A pattern whose entry point answers
 * AIONHIP_UNSUPPORTED for the shape runs as the next smaller pattern or as separate steps. aion folds at step level the same
 * way (graph/opt/fuse_steps.zig:19-88). */
enum { AIONHIP_FUSE_SIBLINGS = 1, AIONHIP_FUSE_WORKSPACE = 2 };
int aionhip_session_set_fusion(aionhip_session *s, int mask);
/* Session.execute (backend/backend.zig:42-44): runs the list in order on the context's stream; asynchronous unless the
 * list holds a device-to-host Transfer, which returns when its bytes have arrived (backend/gpu/backend.zig:416-457). The
 * first use of a MatMul / MatMulNT b builds its re-laid weight from the blocks on the device and keeps it for the session
 * (keyed by address, dtype and shape: retire the session before a weight tensor's storage is released or reused, which is
 * when the reference calls retireResources). May run between aionhip_program_begin and aionhip_program_end once the same list
 * has run eagerly (weights built, scratch grown; no Transfer steps then). On failure aionhip_last_error names the step. */
int aionhip_session_execute(aionhip_session *s, const aionhip_step *steps, size_t count);
/* launches the last execute made (a folded pattern counts as its calls) and re-laid weights the session holds */
int aionhip_session_stats(const aionhip_session *s, uint64_t *calls_last_execute, uint64_t *weights, uint64_t *weight_bytes);
/* Session.retireResources (backend/backend.zig:36-38): waits for the stream and drops what may retain tensor backings -
 * the re-laid weights and the bf16 copies the context made of them. The session stays usable. */
int aionhip_session_retire(aionhip_session *s);
void aionhip_session_destroy(aionhip_session *s);     /* Session.deinit; retires first */

/* ---- timing helpers for the roofline harness (timestamp queries of the WebGPU backend,
 *      backend/gpu/timestamp_profile.zig, reduced to stream events) ------------------------- */
int aionhip_event_create(aionhip_ctx *ctx, void **event);
int aionhip_event_record(aionhip_ctx *ctx, void *event);
int aionhip_event_elapsed_ms(aionhip_ctx *ctx, void *start, void *stop, float *ms); /* waits for `stop` */
void aionhip_event_destroy(aionhip_ctx *ctx, void *event);

/* Per-launch GPU timing of the matmul / attention kernels (AION_PROFILE_GPU=dispatch in the
 * WebGPU backend, backend/gpu/timestamp_profile.zig:1-60): between start and stop every such
 * launch carries its own start and stop event (the dispatch's timestamps, as a kernel trace
 * reports them); stop waits for the stream and resolves them. */
int aionhip_profile_start(aionhip_ctx *ctx);
int aionhip_profile_stop(aionhip_ctx *ctx, size_t *count);
int aionhip_profile_entry(aionhip_ctx *ctx, size_t index, const char **name, float *ms);

#ifdef __cplusplus
}
#endif
#endif /* AION_HIP_H */
