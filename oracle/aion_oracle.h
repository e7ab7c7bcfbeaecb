/* CPU oracle for the aion quantized-inference hot path.
 *
 * TEST INFRASTRUCTURE ONLY. This is a scalar restatement of the arithmetic of
 * RubyBit/aion's CPU kernels (Zig), used to check the HIP kernels and, timed,
 * as the "reference-algorithm CPU baseline". Nothing shipped links or loads it.
 *
 * Every function cites the reference file:line (relative to the aion source
 * tree) whose arithmetic it follows. Integer parts (block codes, int8 dots) are
 * exact restatements; f32 accumulation order is fixed to ONE admissible order of
 * the reference (its SIMD lane folding depends on the host ISA tier), which only
 * moves results at the 1e-7 relative level.
 *
 * Pinning status (what independent check fixes each function):
 *   orc_quantize_q8 / q4        reference in-test inputs (storage/quantize.zig:105-137,
 *                               api/test_api.zig:4660-4700) + closed-form special cases
 *                               (zero block, +-absmax, rounding ties) + numpy float16 RNE.
 *   orc_prepare_a               brute force against the closed form; signed/unsigned dot identity.
 *   orc_matmul_nt_q8, orc_matmul_q8_kmajor, orc_matmul_q4_kmajor
 *                               f64 evaluation of sum(a_s*b_s*idot) on the reference tests'
 *                               closed-form inputs (matvec_q.zig:176-219, matmul_nt_q.zig:587-637),
 *                               dequantized f32 matmul on tiny shapes, strided==compact invariant.
 *   orc_attention_blocked       textbook f64 softmax attention (orc_attention_f64), torch SDPA on
 *                               causal cases, hand-computable KATs (api/test_api.zig:3256-3331,
 *                               api/test_nn.zig:799-901), split==unsplit invariant.
 *   glue (rmsnorm, rope, gate, gather, cast, append, argmax): closed forms in numpy.
 *   matmul_nt_f32 (oracle.py, numpy; cpu/kernels/matmul_nt.zig:40-126): the float64 product within the bound K fixes,
 *                               and bit equality on inputs whose partial sums are all exact in f32.
 */
#ifndef AION_ORACLE_H
#define AION_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORC_Q8_0 = 4, ORC_Q4_0 = 3 }; /* aion DType ids: backend/types.zig:29-39 */

/* f16 <-> f32 (IEEE binary16, round to nearest even; Zig @floatCast). */
uint16_t orc_f32_to_f16(float v);
float orc_f16_to_f32(uint16_t bits);

/* storage/quantize.zig:31-103 (q8_0) and cpu/test_cpu_kernels.zig:490-523 (q4_0).
 * shape[rank] row-major f32 -> packed blocks, row-major over block space.
 * Returns 0, or -1 on InvalidArgument (axis not a multiple of 32, bad rank). */
int orc_quantize(int dtype, const size_t *shape, size_t rank, size_t quant_axis,
                 const float *values, uint8_t *out);
/* inverse: blocks -> f32 row-major of `shape` (q4 decode: matmul_q_i8.zig:362-370) */
int orc_dequantize(int dtype, const size_t *shape, size_t rank, size_t quant_axis,
                   const uint8_t *blocks, float *out);

/* matmul_q_i8.zig:187-203,227-264: int8 activation per (row, 32-block).
 * aq[m][k] int8, a_scale[m][k/32] f32, a_sum[m][k/32] i32 (plain sum of the codes). */
void orc_prepare_a(const float *a, size_t m, size_t k, size_t lda,
                   int8_t *aq, float *a_scale, int32_t *a_sum);

/* cpu/kernels/matmul_nt_q.zig:74-95,173-216 + exec/matmul_nt.zig:87-259.
 * C[m,n] = alpha * A[m,k] @ B[n,k]^T + beta*C; B q8_0 blocks [n][k/32] (34 B). */
int orc_matmul_nt_q8(size_t m, size_t n, size_t k, float alpha, float beta,
                     const float *a, size_t lda, const uint8_t *b_blocks,
                     float *c, size_t ldc, int threads);

/* cpu/kernels/matvec_q.zig:62-160: B q8_0 blocks [k/32][ldb] (K-major), K in chunks of 8192. */
int orc_matmul_q8_kmajor(size_t m, size_t n, size_t k, float alpha, float beta,
                         const float *a, size_t lda, const uint8_t *b_blocks, size_t ldb,
                         float *c, size_t ldc, int threads);

/* cpu/kernels/matmul_q_i8.zig:314-497 + exec/matmul.zig:381-463: packed int8 GEMM,
 * B q4_0 or q8_0 blocks [k/32][n] (K-major); K walked in `kc` steps (128|256|512). */
int orc_matmul_q_packed(int dtype, size_t m, size_t n, size_t k, float alpha, float beta,
                        const float *a, size_t lda, const uint8_t *b_blocks,
                        float *c, size_t ldc, size_t kc, int threads);

/* "f32-A dequant" family (backend/gpu/test_gpu_backend.zig:1325-1341):
 * C = alpha * A @ deq(B) + beta*C with A kept in f32, accumulated in f64.
 * nt != 0: B is [n][k/32] blocks; nt == 0: B is [k/32][n] blocks. */
int orc_matmul_q_f32a(int dtype, int nt, size_t m, size_t n, size_t k, float alpha, float beta,
                      const float *a, size_t lda, const uint8_t *b_blocks,
                      float *c, size_t ldc, int threads);

/* Attention. Layouts (graph/graph.zig:365-393): q [B,L,Hq,Dk] f32, k [B,T,Hkv,Dk],
 * v [B,T,Hkv,Dv] (kv_dtype: 0 f32, 1 f16 bits), out f32 [B,L,Hq,Dv].
 * window {left,right,chunk} with 0xFFFFFFFF = unbounded (graph/graph.zig:130-181).
 * positions [B,L] i32 or NULL, kv_lengths [B] i32 or NULL. */
typedef struct {
    size_t batch, l_q, t_kv, h_q, h_kv, d_k, d_v;
    float scale, soft_cap;
    uint32_t win_left, win_right, win_chunk;
    int kv_dtype;
} orc_attn_shape;

/* cpu/exec/attention.zig:627-815,1347-1442 + kernels/attention.zig:446-527 + fast_math.zig:53-92:
 * blocked online softmax (row_block 32, key_block 256), polynomial exp. segs>1 splits each
 * unit's key range and LSE-merges (attention.zig:879-962). */
int orc_attention_blocked(const orc_attn_shape *s, const float *q, const void *k, const void *v,
                          const int32_t *positions, const int32_t *kv_lengths, float *out, int segs);
/* textbook f64 softmax(QK^T*scale)V over the same interval window
 * (cachedGqaRefF32, cpu/test_cpu_backend.zig:4806-4900). */
int orc_attention_f64(const orc_attn_shape *s, const float *q, const void *k, const void *v,
                      const int32_t *positions, const int32_t *kv_lengths, float *out);

/* fast_math.zig:79-92, 94-148 */
float orc_exp_approx(float x);
float orc_tanh_approx(float x);

/* glue for the decoder (cpu/exec/layernorm.zig:54-155, kernels/layernorm.zig:7-147):
 * out = x * rsqrt(mean(x^2)+eps) * gamma + beta (+ residual) */
void orc_rmsnorm(const float *x, const float *gamma, const float *beta, const float *residual,
                 size_t rows, size_t cols, float eps, float *out);
/* cpu/exec/rope.zig:14-53, kernels/rope.zig:20-98: x [B,T,H,D], positions [B,T] */
void orc_rope(const float *x, const int32_t *positions, size_t b, size_t t, size_t h, size_t d,
              float base, float scale_factor, float proportion, float *out);
/* cpu/exec/elementwise.zig:25-37, kernels/gelu.zig:8-14: out = gelu_tanh_approx(a) * b */
void orc_gate_gelu(const float *a, const float *b, size_t n, float *out);
/* cpu/exec/unary.zig:55-64 over cpu/kernels/{relu,gelu,silu,sigmoid,tanh}.zig and fast_math.zig:53-148; op = UnaryOp id
 * (backend/types.zig:119-125: relu 0, gelu 1, silu 2, sigmoid 3, tanh 4, sqrt 5). Pinned by definition checks, by
 * gelu(a) * b == orc_gate_gelu(a, b) bit for bit and by the approximations' distance from the true functions
 * (tests/test_graph_oracle.py). -1: unknown op */
int orc_unary(int op, const float *x, size_t n, float *out);
/* cpu/exec/elementwise.zig:38-60: add 0 / sub 1 / mul 2 / div 3 with b identical, scalar or a contiguous suffix of a's
 * shape (nb elements, nb divides n): out[i] = a[i] op b[i % nb]. Pinned against numpy broadcasting. -1: invalid */
int orc_binary(int op, const float *a, const float *b, size_t n, size_t nb, float *out);
/* cpu/exec/gather.zig:60-87: rows of a q8_0 [V,D] axis-1 table (or f32 when dtype==0) */
void orc_gather_rows(int dtype, const void *table, size_t d, const int32_t *ids, size_t n_ids, float *out);
/* cpu/exec/argmax.zig:56-81: first maximum wins */
void orc_argmax(const float *x, size_t rows, size_t n, int32_t *out);
void orc_cast_f32_f16(const float *x, size_t n, uint16_t *out);

/* Synthetic decoder (config 5), run entirely with the functions above; see oracle header of
 * the .cpp for the step list (pattern of src/bench/models.zig:433-536). Weights q4_0 [K,N]
 * axis 0 (or q8_0 [N,K] axis 1 when wdtype == ORC_Q8_0); embedding f32 [V,hidden]. */
typedef struct {
    size_t layers, hidden, heads, kv_heads, head_dim, ffn, vocab, max_seq;
    float eps, rope_base;
    int wdtype;
    int attn_exact; /* 0: blocked attention with the polynomial exp (aion's CPU path); 1: textbook f64
                       softmax - used to measure how far the CPU path itself moves under a 4e-5 change */
} orc_decoder_cfg;
typedef struct orc_decoder orc_decoder;
orc_decoder *orc_decoder_create(const orc_decoder_cfg *cfg, int threads);
void orc_decoder_destroy(orc_decoder *d);
/* names: "embed" (f32), per layer l: "l%u.{wq,wk,wv,wo,wgate,wup,wdown}" (blocks),
 * "l%u.{norm1,norm2}" (f32 gamma), "norm_f", "lm_head". Data is copied. */
int orc_decoder_set_weight(orc_decoder *d, const char *name, const void *data, size_t bytes);
void orc_decoder_reset(orc_decoder *d);
/* runs `s` tokens at positions [pos0, pos0+s); logits [s, vocab] (may be NULL -> only last
 * row's argmax returned). Returns argmax of the last row, or -1 on error. */
int32_t orc_decoder_forward(orc_decoder *d, const int32_t *tokens, size_t s, size_t pos0, float *logits_last);

#ifdef __cplusplus
}
#endif
#endif
