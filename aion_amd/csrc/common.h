// Internal declarations shared by the HIP sources of libaion_hip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_ext.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

#include "../../include/aion_hip.h"

using u32x4 = __attribute__((ext_vector_type(4))) unsigned int;   // one 16-byte global load
using f32x4 = __attribute__((ext_vector_type(4))) float;

constexpr int QK = 32;        // elements per quant block (aion backend/types.zig:40-50)
constexpr int Q8_BYTES = 34;  // f16 scale + 32 x i8
constexpr int Q4_BYTES = 18;  // f16 scale + 16 nibble bytes

// One timed kernel launch (per-dispatch GPU timestamps, as aion's WebGPU backend collects with
// AION_PROFILE_GPU=dispatch, backend/gpu/timestamp_profile.zig).
struct ProfRecord {
    const char *name;
    hipEvent_t start, stop;
    float ms;
};

struct aionhip_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    bool own_stream = false;
    std::string err;
    const char *last_kernel = "";
    int gemm_mode = AIONHIP_GEMM_EXACT_I8;
    int cu_count = 0;
    // Device memory pool behind aionhip_alloc / aionhip_free. A freed block of up to POOL_MAX_BLOCK bytes is kept under
    // its size class and handed out again to the next request of that class: everything this context does runs on one
    // stream, so the reuse is ordered behind the last use without the device-wide wait a hipFree implies.
    static constexpr size_t POOL_MAX_BLOCK = (size_t)64 << 20;
    std::unordered_map<void *, size_t> pool_live;                  // block -> bytes of its size class
    std::unordered_map<size_t, std::vector<void *>> pool_free;     // size class -> cached blocks
    size_t pool_live_bytes = 0, pool_cached_bytes = 0;
    // prepared-activation scratch (int8 codes, per-block f32 scale, per-block code sum)
    void *scratch = nullptr;
    size_t scratch_bytes = 0;
    // second scratch for GEMM staging (dequantized weights / bf16 activations / split-K partials)
    void *scratch2 = nullptr;
    size_t scratch2_bytes = 0;
    // K-split GEMV: the words in which the partial sums of sibling K slices meet (all zero between launches)
    void *ksplit = nullptr;
    size_t ksplit_bytes = 0;
    // argmax: one ticket per row (all zero between launches)
    void *tickets = nullptr;
    size_t tickets_bytes = 0;
    // moves on whenever one of the four buffers above is replaced by a larger one: a program recorded before that holds
    // the old address and may not run any more
    uint64_t buffer_generation = 0;
    // this device's copy of the library's file-scope scratch array (ctx.hip), for the entry point that allocates nothing
    void *static_scratch = nullptr;
    // bf16 mode of the GEMM: this context's bf16 copies of the weights it has multiplied (weight -> {copy, bytes}), built
    // on a weight's first bf16 call, released by aionhip_weight_drop_bf16 / aionhip_weight_free / aionhip_destroy;
    // bf16_copies_on = false: no copies, the kernel converts the quant blocks while it stages them
    std::unordered_map<const struct aionhip_weight *, std::pair<void *, size_t>> bf16_copies;
    size_t bf16_copy_bytes = 0;
    bool bf16_copies_on = true;
    // true while that entry point runs: no launcher may take a path that needs scratch of its own
    bool no_scratch_paths = false;
    // attention with f32 queries: false = one MFMA pass on q rounded to the K/V element type (2e-3 class),
    // true = q and the probabilities as hi+lo parts (f32-level accuracy, about 1.4x the instructions)
    bool attn_precise = false;
    // RoPE frequency tables (f32, multiplied up iteratively as on the CPU), one per (pairs, base, d, scale)
    struct RopeTable {
        int pairs;
        float freq_step, scale_factor;
        float *freq;
    };
    std::vector<RopeTable> rope_tables;
    // true between aionhip_program_begin/end: launches are captured, nothing may synchronise or allocate
    bool capturing = false;
    // per-launch timing, off by default
    bool profiling = false;
    const char *prof_name = nullptr;   // set by ProfScope: launches made through launch_k are timed under it
    // the last launch made through launch_k: host stub, grid and block (reports match them to a kernel trace)
    const void *last_fn = nullptr;
    unsigned last_grid[3] = {0, 0, 0}, last_block[3] = {0, 0, 0}, last_lds = 0;
    std::vector<ProfRecord> prof;
    std::vector<hipEvent_t> event_pool;
};

// LDS-writing global loads (global_load_lds_dwordx4) take an address-space-3 destination and are
// waited for by count: s_waitcnt immediate for "vmcnt <= n" only (gfx9 encoding: bits 3:0 and 15:14).
typedef __attribute__((address_space(3))) void lds_void;
constexpr int vmcnt_imm(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

// Names the launches made through launch_k while it is alive (and profiling is on).
struct ProfScope {
    aionhip_ctx *ctx;
    const char *prev;
    ProfScope(aionhip_ctx *c, const char *name) : ctx(c), prev(c->prof_name) { c->prof_name = name; }
    ~ProfScope() { ctx->prof_name = prev; }
};
// A new profile record under the scope's name; its two events go to the launch.
void prof_open(aionhip_ctx *ctx, hipEvent_t *start, hipEvent_t *stop);

// Kernel launch on the context's stream. While profiling inside a ProfScope the launch carries its
// own start/stop events (hipExtLaunchKernelGGL: the timestamps of the dispatch itself, so the
// elapsed time is the kernel's duration with no barrier or launch gap in it).
template <typename... KArgs, typename... Args>
inline void launch_k(aionhip_ctx *ctx, void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds, Args... args) {
    ctx->last_fn = (const void *)kernel;
    ctx->last_grid[0] = grid.x, ctx->last_grid[1] = grid.y, ctx->last_grid[2] = grid.z;
    ctx->last_block[0] = block.x, ctx->last_block[1] = block.y, ctx->last_block[2] = block.z;
    ctx->last_lds = (unsigned)lds;
    if (ctx->profiling && ctx->prof_name) {
        hipEvent_t e0 = nullptr, e1 = nullptr;
        prof_open(ctx, &e0, &e1);
        hipExtLaunchKernelGGL(kernel, grid, block, (uint32_t)lds, ctx->stream, e0, e1, 0u, static_cast<KArgs>(args)...);
    } else {
        kernel<<<grid, block, lds, ctx->stream>>>(static_cast<KArgs>(args)...);
    }
}

// Device-private weight layout: row n of the [N,K] operand is one contiguous run.
//   q8_0: qs[n][K] int8,               sc[n][K/32] f16
//   q4_0: qs[n][K/2] nibble bytes,     sc[n][K/32] f16
// q4 nibble order inside each 32-bit word (8 elements e0..e7): byte i = e[i] | e[4+i] << 4, so
// (w & 0x0F0F0F0F) is elements 0..3 and ((w >> 4) & 0x0F0F0F0F) is elements 4..7, each directly
// usable as the byte operand of a 4-way int8 dot.
struct aionhip_weight {
    int dtype = 0;
    int layout = 0;
    size_t n = 0, k = 0;
    uint8_t *qs = nullptr;
    __half *sc = nullptr;
    size_t qs_bytes = 0, sc_bytes = 0;
};

int set_err(aionhip_ctx *ctx, int status, const char *fmt, ...);
int dev_malloc(aionhip_ctx *ctx, void **out, size_t bytes, const char *what);
int grow_work_buffer(aionhip_ctx *ctx, void **buf, size_t *have, size_t bytes, bool zeroed, const char *what);
int ensure_scratch(aionhip_ctx *ctx, size_t bytes);
int ensure_scratch2(aionhip_ctx *ctx, size_t bytes);
// size of the file-scope device scratch array behind aionhip_step_matmul_static (prepared activations of one call)
constexpr size_t STATIC_SCRATCH_BYTES = AIONHIP_STATIC_SCRATCH_BYTES;

#define HIP_TRY(ctx, expr)                                                                          \
    do {                                                                                            \
        hipError_t e_ = (expr);                                                                     \
        if (e_ != hipSuccess)                                                                       \
            return set_err((ctx), e_ == hipErrorOutOfMemory ? AIONHIP_OUT_OF_MEMORY : AIONHIP_EXECUTION_FAILED, \
                           "%s: %s", #expr, hipGetErrorString(e_));                                 \
    } while (0)

#define LAUNCH_CHECK(ctx, name)                                                                     \
    do {                                                                                            \
        (ctx)->last_kernel = (name);                                                                \
        hipError_t e_ = hipGetLastError();                                                          \
        if (e_ != hipSuccess) return set_err((ctx), AIONHIP_EXECUTION_FAILED, "launch %s: %s", (name), hipGetErrorString(e_)); \
    } while (0)

// ---- prepared activations (aion cpu/kernels/matmul_q_i8.zig:187-264) --------------------------
struct PreparedAct {
    int8_t *q;      // [m][k]
    float *scale;   // [m][k/32]
    int *sum;       // [m][k/32]   plain sum of the 32 codes
};
size_t prepared_act_bytes(size_t m, size_t k);
PreparedAct prepared_act_carve(void *base, size_t m, size_t k);
int launch_prepare_act(aionhip_ctx *ctx, const float *a, size_t lda, size_t m, size_t k, PreparedAct out);
int launch_prepare_gate(aionhip_ctx *ctx, const float *gate, const float *up, size_t m, size_t k, PreparedAct out);
int launch_prepare_rmsnorm(aionhip_ctx *ctx, const float *x, const float *gamma, const float *beta, float eps, size_t m, size_t k, PreparedAct out);

// ---- matmul back ends --------------------------------------------------------------------------
// Up to four weights that multiply the SAME activation rows (q/k/v, gate/up) run as one launch:
// their rows are concatenated, a wavefront's row group never straddles two weights.
struct GemvSeg {
    const u32x4 *qs;
    const __half *sc;
    float *c;
    size_t ldc;
    int n;          // rows of this weight
    int first_wave; // first wavefront of this segment
};
struct GemvBatch {
    GemvSeg seg[4];
    int count;
    int total_waves;
};
// What the single-row GEMV computes its activation from, inside the kernel (no separate launch):
//   PRO_QUANT   a = x
//   PRO_RMSNORM a = x * rsqrt(mean(x^2)+eps) * gamma + beta
//   PRO_GATE    a = gelu_tanh(x) * y
enum { PRO_QUANT = 0, PRO_RMSNORM = 1, PRO_GATE = 2 };
struct FusedIn {
    const float *x, *y, *gamma, *beta;
    float eps;
};
// Optional epilogue of the single-row GEMV. EPI_ROPE_APPEND: the three weights are Wq, Wk, Wv of one
// attention block; a wavefront owns the rows e..e+3 and e+D/2..e+D/2+3 of one head, i.e. both halves
// of four RoPE pairs, rotates them (q, k) and writes q as f32 and k, v as f16 rows of the KV cache at
// the device-resident write index: the q/k/v GEMV, RoPE, the f16 cast and the cache append in one launch.
// EPI_GATE_QUANT: the two weights are the gate and up projections of a GeGLU block; a workgroup owns 32
// consecutive outputs j of both (a wavefront: rows j..j+3 of each, twice), forms h_j = gelu_tanh(g_j) * u_j
// and writes the block's int8 activation preparation (codes, scale, code sum) for the down projection:
// neither g, u nor h goes to memory and no separate gate / preparation launch is needed.
enum { EPI_NONE = 0, EPI_ROPE_APPEND = 1, EPI_GATE_QUANT = 2 };
struct FusedEpi {
    const int *positions, *write_index;
    const float *freq;
    __half *k_cache, *v_cache;
    int t_cap, h_kv, d, rope_pairs;
    int rolling;         // the caches are rings: logical step t lives in row t % t_cap
    int *act_q;          // EPI_GATE_QUANT: prepared activation planes of the down projection
    float *act_scale;
    int *act_sum;
};
constexpr size_t FUSED_MAX_K = 8192;
// above this K the per-workgroup prologue costs more than a separate preparation launch
constexpr size_t FUSED_PAYS_K = 4096;
int launch_gemv_fused(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count,
                      int prologue, FusedIn in, float alpha, float beta);
int launch_gemv_fused_rope(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *q_out, FusedIn in, FusedEpi epi);
int launch_gemv_fused_geglu(aionhip_ctx *ctx, const aionhip_weight *gate, const aionhip_weight *up, FusedIn in, PreparedAct out);
int launch_rmsnorm(aionhip_ctx *ctx, float *out, const float *x, const float *gamma, const float *beta, const float *residual,
                   size_t rows, size_t cols, float eps);
int launch_gate_gelu(aionhip_ctx *ctx, float *out, const float *a, const float *b, size_t n);
// device table f[i] = scale_factor * freq_step^i built with f32 multiplies in sequence (aion cpu/kernels/rope.zig:22-30)
int rope_table(aionhip_ctx *ctx, int pairs, float freq_step, float scale_factor, const float **out);

// one activation row against one weight with a long reduction axis: K cut into slices, one launch (gemv_ksplit.hip)
// 3..8 prepared rows against a weight with very many rows, the dots on the matrix pipe (gemv_mfma.hip); launch returns -1 when
// the shape does not suit the kernel after all
bool gemv_mfma_applies(const aionhip_weight *const *ws, int count, int m);
int launch_gemv_mfma(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, int m, PreparedAct act,
                     float alpha, float beta);
bool gemv_ksplit_applies(const aionhip_ctx *ctx, const aionhip_weight *w, const float *x);
int launch_gemv_ksplit(aionhip_ctx *ctx, const aionhip_weight *w, float *c, const float *x, float alpha, float beta);
int launch_gemv(aionhip_ctx *ctx, const aionhip_weight *w, int m, PreparedAct act, float *c, size_t ldc, float alpha, float beta);
int launch_gemv_batch(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, int m,
                      PreparedAct act, float alpha, float beta);
int launch_gemm_i8(aionhip_ctx *ctx, const aionhip_weight *w, size_t m, PreparedAct act, float *c, size_t ldc, float alpha, float beta);
// bf16 mode only: whether the bf16 MFMA kernel is expected to be the faster one for m rows against an n x k weight
bool gemm_bf16_pays(const aionhip_ctx *ctx, size_t m, size_t n, size_t k);
// the LDS-staged MFMA kernel for a handful of rows (no profile scope of its own: the caller's name stays)
int launch_gemm_i8_batch(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, size_t m,
                         PreparedAct act, float alpha, float beta);
int launch_gemm_i8_few_rows(aionhip_ctx *ctx, const aionhip_weight *w, size_t m, PreparedAct act, float *c, size_t ldc, float alpha, float beta);
// MatMulNT with an f32 [N,K] operand (matmul_nt_f32.hip): plain f32 arithmetic, any number of rows
int launch_matmul_nt_f32(aionhip_ctx *ctx, const aionhip_weight *w, size_t m, const float *a, size_t lda, float *c, size_t ldc, float alpha,
                         float beta);
int launch_gemm_bf16(aionhip_ctx *ctx, const aionhip_weight *w, size_t m, const float *a, size_t lda, float *c, size_t ldc, float alpha, float beta);

// ---- wave64 cross-lane helpers -----------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
constexpr int DPP_QUAD_XOR1 = 0xB1;     // quad_perm [1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;     // quad_perm [2,3,0,1]
constexpr int DPP_ROW_HALF_MIRROR = 0x141;
constexpr int DPP_ROW_MIRROR = 0x140;

// The rotation of one RoPE pair with every product and the sum rounded on its own, as aion's CPU kernel computes it
// (cpu/kernels/rope.zig:90-91, no fused multiply-add) - and so the same bits from every kernel that rotates.
__device__ __forceinline__ void rope_rotate(float xl, float xh, float sn, float cs, float &yl, float &yh) {
#pragma clang fp contract(off)
    yl = xl * cs - xh * sn;
    yh = xl * sn + xh * cs;
}

// sum over the 64 lanes of a wavefront; every lane returns the total
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f<DPP_QUAD_XOR1>(v);
    v += dpp_f<DPP_QUAD_XOR2>(v);
    v += dpp_f<DPP_ROW_HALF_MIRROR>(v);
    v += dpp_f<DPP_ROW_MIRROR>(v);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_f<DPP_QUAD_XOR1>(v));
    v = fmaxf(v, dpp_f<DPP_QUAD_XOR2>(v));
    v = fmaxf(v, dpp_f<DPP_ROW_HALF_MIRROR>(v));
    v = fmaxf(v, dpp_f<DPP_ROW_MIRROR>(v));
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}

// The int8 preparation of one 32-element activation block (aion cpu/kernels/matmul_q_i8.zig:187-203 quantizeABlock,
// :227-264 prepareARow) held by 8 consecutive lanes, 4 values each: amax over the block; a zero block gives zero
// codes and scale 0; else scale = amax / 127, inv = 127 / amax, code = clamp(round-half-away(v * inv), -127, 127).
// Every lane of the 8 returns its four codes packed into `word`, the block scale and the plain sum of the 32 codes.
// The one definition every kernel that prepares activations calls, so that they cannot drift apart.
__device__ __forceinline__ void prepare_act_block8(float v0, float v1, float v2, float v3, int &word, float &scale, int &sum) {
    float amax = fmaxf(fmaxf(fabsf(v0), fabsf(v1)), fmaxf(fabsf(v2), fabsf(v3)));
    amax = fmaxf(amax, dpp_f<DPP_QUAD_XOR1>(amax));
    amax = fmaxf(amax, dpp_f<DPP_QUAD_XOR2>(amax));
    amax = fmaxf(amax, dpp_f<DPP_ROW_HALF_MIRROR>(amax));
    word = 0;
    scale = 0.f;
    int s = 0;
    if (amax != 0.f) {
        scale = amax / 127.f;
        const float inv = 127.f / amax;
        const int q0 = (int)fminf(127.f, fmaxf(-127.f, roundf(v0 * inv)));
        const int q1 = (int)fminf(127.f, fmaxf(-127.f, roundf(v1 * inv)));
        const int q2 = (int)fminf(127.f, fmaxf(-127.f, roundf(v2 * inv)));
        const int q3 = (int)fminf(127.f, fmaxf(-127.f, roundf(v3 * inv)));
        word = (q0 & 0xFF) | ((q1 & 0xFF) << 8) | ((q2 & 0xFF) << 16) | ((q3 & 0xFF) << 24);
        s = q0 + q1 + q2 + q3;
    }
    s += dpp_i<DPP_QUAD_XOR1>(s);
    s += dpp_i<DPP_QUAD_XOR2>(s);
    s += dpp_i<DPP_ROW_HALF_MIRROR>(s);
    sum = s;
}

__device__ __forceinline__ int dot4_i8(int a, int b, int c) { return __builtin_amdgcn_sdot4(a, b, c, false); }

// aion cpu/kernels/fast_math.zig:53-148: exp(x) = 2^n * P4(r ln2), sigmoid, tanh = 2 sigmoid(2x) - 1
__device__ __forceinline__ float aion_exp_approx(float x_in) {
    const float x = fminf(80.f, fmaxf(-80.f, x_in));
    const float y = x * 1.4426950408889634f;
    const float nf = floorf(y + 0.5f);
    const float t = (y - nf) * 0.6931471805599453f;
    const float p = 1.f + t * (1.f + t * (0.5f + t * ((1.f / 6.f) + t * (1.f / 24.f))));
    return __uint_as_float((unsigned)((int)nf + 127) << 23) * p;
}
__device__ __forceinline__ float aion_tanh_approx(float x) {
    const float z = 2.f * x;
    const float e = aion_exp_approx(-fabsf(z));
    float sg = (z >= 0.f ? 1.f : e) / (1.f + e);
    sg = fminf(1.f, fmaxf(0.f, sg));
    return fminf(1.f, fmaxf(-1.f, 2.f * sg - 1.f));
}
__device__ __forceinline__ float aion_sigmoid_approx(float x) {
    const float e = aion_exp_approx(-fabsf(x));
    return fminf(1.f, fmaxf(0.f, (x >= 0.f ? 1.f : e) / (1.f + e)));
}
// aion cpu/exec/elementwise.zig:25-37 (gate) + cpu/kernels/gelu.zig:8-14: gelu_tanh(x) * up
__device__ __forceinline__ float aion_gate_gelu(float x, float up) {
    const float t = 0.7978845608028654f * (x + 0.044715f * (x * x * x));
    return (0.5f * x * (1.f + aion_tanh_approx(t))) * up;
}
// sum over a 256-thread workgroup; red: 4 floats of LDS. Every thread returns the total.
__device__ __forceinline__ float block_sum_256(float v, float *red) {
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    const float t = (red[0] + red[1]) + (red[2] + red[3]);
    __syncthreads();
    return t;
}
