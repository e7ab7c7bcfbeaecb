// StepMatMul / StepMatMulNT entry points: argument checks (the aion compiler's validation,
// graph/program/compiler.zig:189-239,337-357), activation preparation, kernel routing
// (the counterpart of cpu/exec/matmul.zig:233-296 `matvecRoute` / `gemm2D`):
//   m == 1, k <= 4096, 16-byte aligned A  -> gemv_fused_kernel (activation prepared in the kernel)
//   m <= 8                                -> prepare_act_kernel + gemv_kernel / gemv_rows_kernel (5..8 rows against a
//                                            wide short weight: the 16-row tile of gemm_i8_lds_kernel)
//   m  > 8                                -> gemm_i8_lds_kernel (exact) or gemm_bf16_wide_kernel
// and the decode fusions built on the single-row kernel: RMSNorm / gelu-gate prologues, the q/k/v + RoPE +
// cache-append launch and the GeGLU block (two launches).
#include "common.h"

#include <cstring>

#include <cmath>

namespace {

constexpr size_t GEMV_MAX_M = 8;

struct Batch {
    size_t count = 0, k = 0;
    const aionhip_weight *w[4];
    float *c[4];
    size_t ldc[4];
    aionhip_handle c_h[4];
};

int check_batch(aionhip_ctx *ctx, const char *what, size_t count, const aionhip_weight *const *bs, const aionhip_handle *c_hs,
                const size_t *ldcs_in, Batch &out) {
    if (count == 0 || count > 4) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "%s: 1..4 weights per call", what);
    if (!bs || !c_hs) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "%s: null argument", what);
    out.count = count;
    out.k = bs[0] ? bs[0]->k : 0;
    for (size_t i = 0; i < count; ++i) {
        if (!bs[i] || !c_hs[i]) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "%s: null weight or C", what);
        if (bs[i]->k != out.k || bs[i]->dtype != bs[0]->dtype) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "%s: weights must share k and dtype", what);
        // an f32 weight is the operand of the plain MatMulNT step only: the fused and batched steps are built on block dots
        if (bs[i]->dtype == AIONHIP_F32 && (count != 1 || strcmp(what, "matmul") != 0))
            return set_err(ctx, AIONHIP_UNSUPPORTED, "%s: f32 weights run as single MatMulNT steps", what);
        out.ldc[i] = ldcs_in && ldcs_in[i] ? ldcs_in[i] : bs[i]->n;
        if (out.ldc[i] < bs[i]->n || (c_hs[i] & 3)) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "%s: ldc below n, or C not 4-byte aligned", what);
        out.w[i] = bs[i];
        out.c[i] = (float *)(uintptr_t)c_hs[i];
        out.c_h[i] = c_hs[i];
    }
    return AIONHIP_OK;
}

// One row: the kernel that prepares the activation in every workgroup. Up to FUSED_PAYS_K always; up to FUSED_MAX_K where
// the outputs are many enough for the weight stream to hide the longer prologue (from 16384 outputs on it measures 8-30 %
// ahead of both the K slices and preparation + GEMV: q4 8192 -> 28672 at 23.2 against 25.3 us, q8 8192 -> 32768 at 46 against 65),
// up to a GiB of weights (q8 8192 -> 131072, 1.14 GB, measures 207 against 175 us the other way).
// Sibling weights in one call have no K-slice form: up to FUSED_MAX_K they stay here as well, one launch against preparation +
// GEMV (q/k/v of 5120 -> 5120 + 2 x 1024, q4: 6.5 against 10.2 us; 8192 -> 8192 + 2 x 1024: 11.0 against 18.2).
static bool fused_row_pays(const Batch &b) {
    if (b.k <= FUSED_PAYS_K) return true;
    if (b.count > 1 && b.k <= FUSED_MAX_K) return true;
    size_t n = 0;
    for (size_t i = 0; i < b.count; ++i) n += b.w[i]->n;
    const size_t bytes = n * (b.k / 32) * (b.w[0]->dtype == AIONHIP_Q8_0 ? 34 : 18);
    return b.k <= FUSED_MAX_K && n >= 16384 && bytes <= ((size_t)1 << 30);
}

// Prepared rows against the weights of `b`: the GEMV kernels up to eight rows, except five to eight rows over a K past 4096,
// where the GEMV walks K with all eight accumulator sets live and falls far behind the exact GEMM's 16-row tile (q8
// 14336 x 8192 at 8 rows: 80 against 33 us, q4 65 against 29; the two meet at K = 4096 ... 5120); the GEMM beyond eight rows.
static int launch_prepared_rows(aionhip_ctx *ctx, const Batch &b, size_t m, PreparedAct act, float alpha, float beta) {
    if (m <= GEMV_MAX_M && !(m >= 5 && b.k > FUSED_PAYS_K))
        return launch_gemv_batch(ctx, b.w, b.c, b.ldc, (int)b.count, (int)m, act, alpha, beta);
    // sibling weights (q/k/v, gate/up) share one launch, four at a time
    for (size_t i = 0; i < b.count; i += 4) {
        const size_t cnt = b.count - i < 4 ? b.count - i : 4;
        const int rc = launch_gemm_i8_batch(ctx, b.w + i, b.c + i, b.ldc + i, (int)cnt, m, act, alpha, beta);
        if (rc) return rc;
    }
    return AIONHIP_OK;
}

// every weight of `b` against the f32 rows at `a` (already materialised). static_scratch: the prepared activation goes
// to the library's file-scope device array and nothing on the way may allocate.
int run_rows(aionhip_ctx *ctx, const Batch &b, size_t m, const float *a, size_t lda, float alpha, float beta, bool static_scratch = false) {
    if (m > 0x7FFFFFFFu) return set_err(ctx, AIONHIP_UNSUPPORTED, "matmul: m exceeds 2^31-1");
    if (b.w[0]->dtype == AIONHIP_F32) return launch_matmul_nt_f32(ctx, b.w[0], m, a, lda, b.c[0], b.ldc[0], alpha, beta);
    if (static_scratch) {
        if (ctx->profiling) return set_err(ctx, AIONHIP_UNSUPPORTED, "matmul_static: not available while per-launch profiling is on (it creates events)");
        if (m > GEMV_MAX_M && ctx->gemm_mode != AIONHIP_GEMM_EXACT_I8)
            return set_err(ctx, AIONHIP_UNSUPPORTED, "matmul_static: more than %zu rows under a bf16 GEMM mode would allocate", GEMV_MAX_M);
        if (prepared_act_bytes(m, b.k) > STATIC_SCRATCH_BYTES)
            return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "matmul_static: the prepared activation of m=%zu, k=%zu needs %zu bytes, the static scratch holds %zu",
                           m, b.k, prepared_act_bytes(m, b.k), STATIC_SCRATCH_BYTES);
    }
    if (m == 1 && fused_row_pays(b) && ((uintptr_t)a & 15) == 0)
        return launch_gemv_fused(ctx, b.w, b.c, b.ldc, (int)b.count, PRO_QUANT, FusedIn{a, nullptr, nullptr, nullptr, 0.f}, alpha, beta);
    // one row, one weight, long K: slices of K across workgroups, preparation inside, one launch (it keeps a growable buffer
    // of its own, so not on the path that may not allocate)
    if (m == 1 && b.count == 1 && !static_scratch && gemv_ksplit_applies(ctx, b.w[0], a))
        return launch_gemv_ksplit(ctx, b.w[0], b.c[0], a, alpha, beta);
    if (m > GEMV_MAX_M && ctx->gemm_mode != AIONHIP_GEMM_EXACT_I8 && !static_scratch) {
        // the bf16 kernel where it is expected to win (or always, if so asked), the exact kernel (below) for the rest
        bool all_bf16 = true;
        if (ctx->gemm_mode == AIONHIP_GEMM_BF16_MFMA)
            for (size_t i = 0; i < b.count; ++i) all_bf16 = all_bf16 && gemm_bf16_pays(ctx, m, b.w[i]->n, b.k);
        if (all_bf16) {
            for (size_t i = 0; i < b.count; ++i) {
                int rc = launch_gemm_bf16(ctx, b.w[i], m, a, lda, b.c[i], b.ldc[i], alpha, beta);
                if (rc) return rc;
            }
            return AIONHIP_OK;
        }
    }
    int rc = static_scratch ? (int)AIONHIP_OK : ensure_scratch(ctx, prepared_act_bytes(m, b.k));
    if (rc) return rc;
    PreparedAct act = prepared_act_carve(static_scratch ? ctx->static_scratch : ctx->scratch, m, b.k);
    rc = launch_prepare_act(ctx, a, lda, m, b.k, act);
    if (rc) return rc;
    return launch_prepared_rows(ctx, b, m, act, alpha, beta);
}

int run_matmul(aionhip_ctx *ctx, const aionhip_weight *w, size_t m, aionhip_handle a_h, size_t lda, aionhip_handle c_h, size_t ldc,
               float alpha, float beta, bool static_scratch = false) {
    if (m == 0) return AIONHIP_OK;
    if (!a_h || !c_h) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "matmul: null A or C");
    if (lda == 0) lda = w->k;
    if (lda < w->k || (a_h & 3)) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "matmul: lda=%zu below k=%zu, or A not 4-byte aligned", lda, w->k);
    Batch b;
    int rc = check_batch(ctx, "matmul", 1, &w, &c_h, &ldc, b);
    if (rc) return rc;
    return run_rows(ctx, b, m, (const float *)(uintptr_t)a_h, lda, alpha, beta, static_scratch);
}

}  // namespace

extern "C" {

int aionhip_step_matmul_batch(aionhip_ctx *ctx, size_t count, const aionhip_weight *const *bs, size_t m, aionhip_handle a, size_t lda,
                              const aionhip_handle *c, const size_t *ldc, float alpha, float beta) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (count == 0 || m == 0) return AIONHIP_OK;
    Batch b;
    int rc = check_batch(ctx, "matmul_batch", count, bs, c, ldc, b);
    if (rc) return rc;
    if (!a) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "matmul_batch: null A");
    if (lda == 0) lda = b.k;
    if (lda < b.k || (a & 3)) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "matmul_batch: lda below k, or A not 4-byte aligned");
    return run_rows(ctx, b, m, (const float *)(uintptr_t)a, lda, alpha, beta);
}

int aionhip_step_matmul(aionhip_ctx *ctx, const aionhip_weight *b, size_t m, aionhip_handle a, size_t lda,
                        aionhip_handle c, size_t ldc, float alpha, float beta) {
    if (!ctx || !b) return AIONHIP_INVALID_ARGUMENT;
    if (b->layout != AIONHIP_KMAJOR_KN) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "MatMul needs a [K,N] K-blocked weight (quant_axis 0)");
    return run_matmul(ctx, b, m, a, lda, c, ldc, alpha, beta);
}

int aionhip_step_matmul_nt(aionhip_ctx *ctx, const aionhip_weight *b, size_t m, aionhip_handle a, size_t lda,
                           aionhip_handle c, size_t ldc, float alpha, float beta) {
    if (!ctx || !b) return AIONHIP_INVALID_ARGUMENT;
    // StepMatMulNT: B is [N,K], q8_0 with quant_axis 1 or f32 (runtime/executable.zig:211-223, cpu/exec/matmul_nt.zig:100)
    if (b->layout != AIONHIP_ROWS_NK || (b->dtype != AIONHIP_Q8_0 && b->dtype != AIONHIP_F32))
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "MatMulNT needs a q8_0 (quant_axis 1) or f32 [N,K] weight");
    return run_matmul(ctx, b, m, a, lda, c, ldc, alpha, beta);
}

int aionhip_step_matmul_static(aionhip_ctx *ctx, const aionhip_weight *b, size_t m, aionhip_handle a, size_t lda,
                               aionhip_handle c, size_t ldc, float alpha, float beta) {
    if (!ctx || !b) return AIONHIP_INVALID_ARGUMENT;
    if (!ctx->static_scratch) return set_err(ctx, AIONHIP_EXECUTION_FAILED, "matmul_static: the context has no static scratch address");
    ctx->no_scratch_paths = true;
    const int rc = run_matmul(ctx, b, m, a, lda, c, ldc, alpha, beta, true);
    ctx->no_scratch_paths = false;
    return rc;
}

int aionhip_step_rmsnorm_matmul(aionhip_ctx *ctx, size_t count, const aionhip_weight *const *bs, size_t rows, aionhip_handle x,
                                aionhip_handle gamma, aionhip_handle beta_norm, float eps, const aionhip_handle *c, const size_t *ldc,
                                float alpha, float beta) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (count == 0 || rows == 0) return AIONHIP_OK;
    Batch b;
    int rc = check_batch(ctx, "rmsnorm_matmul", count, bs, c, ldc, b);
    if (rc) return rc;
    if (!x || !gamma) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "rmsnorm_matmul: null x or gamma");
    if (!(eps > 0.f) || !(eps < INFINITY)) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "rmsnorm_matmul: eps must be positive and finite");
    const float *xp = (const float *)(uintptr_t)x, *gp = (const float *)(uintptr_t)gamma, *bp = (const float *)(uintptr_t)beta_norm;
    if (rows == 1 && fused_row_pays(b) && ((x | gamma | beta_norm) & 15) == 0)
        return launch_gemv_fused(ctx, b.w, b.c, b.ldc, (int)b.count, PRO_RMSNORM, FusedIn{xp, nullptr, gp, bp, eps}, alpha, beta);
    // Two rows and more on the exact kernels: the norm and the int8 preparation in one launch (the bits of the norm step followed
    // by the preparation launch), then the GEMV or GEMM on the prepared rows. One row keeps the route below (a long K is cut
    // into slices that prepare their own part), and so does a call that the bf16 kernel takes (it wants the f32 rows).
    bool bf16_route = rows > GEMV_MAX_M && ctx->gemm_mode != AIONHIP_GEMM_EXACT_I8;
    if (bf16_route && ctx->gemm_mode == AIONHIP_GEMM_BF16_MFMA)
        for (size_t i = 0; i < b.count; ++i) bf16_route = bf16_route && gemm_bf16_pays(ctx, rows, b.w[i]->n, b.k);
    if (rows >= 2 && rows <= 0x7FFFFFFFu && !bf16_route && ((x | gamma | beta_norm) & 15) == 0) {
        rc = ensure_scratch(ctx, prepared_act_bytes(rows, b.k));
        if (rc) return rc;
        PreparedAct act = prepared_act_carve(ctx->scratch, rows, b.k);
        rc = launch_prepare_rmsnorm(ctx, xp, gp, bp, eps, rows, b.k, act);
        if (rc) return rc;
        return launch_prepared_rows(ctx, b, rows, act, alpha, beta);
    }
    // otherwise the norm runs as its own kernel into scratch, then the ordinary routing
    const size_t act_bytes = (prepared_act_bytes(rows, b.k) + 255) & ~(size_t)255;
    rc = ensure_scratch(ctx, act_bytes + rows * b.k * sizeof(float));
    if (rc) return rc;
    float *h = (float *)((char *)ctx->scratch + act_bytes);
    rc = launch_rmsnorm(ctx, h, xp, gp, bp, nullptr, rows, b.k, eps);
    if (rc) return rc;
    return run_rows(ctx, b, rows, h, b.k, alpha, beta);
}

int aionhip_step_rmsnorm_qkv_rope_append(aionhip_ctx *ctx, const aionhip_weight *wq, const aionhip_weight *wk, const aionhip_weight *wv,
                                         aionhip_handle x, aionhip_handle gamma, aionhip_handle beta_norm, float eps,
                                         aionhip_handle q_out, aionhip_handle k_cache, aionhip_handle v_cache,
                                         aionhip_handle positions, aionhip_handle write_index, size_t t_cap, size_t h_q, size_t h_kv,
                                         size_t d, float base_frequency, float scale_factor, float rope_proportion, int rolling) {
    if (!ctx || !wq || !wk || !wv) return AIONHIP_INVALID_ARGUMENT;
    if (!x || !gamma || !q_out || !k_cache || !v_cache || !positions || !write_index)
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "qkv_rope_append: null operand");
    if (!(eps > 0.f) || !(eps < INFINITY)) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "qkv_rope_append: eps must be positive and finite");
    if (!(base_frequency > 0.f) || !(base_frequency < INFINITY) || !(scale_factor > 0.f) || !(scale_factor < INFINITY) ||
        !(rope_proportion >= 0.f && rope_proportion <= 1.f))
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "qkv_rope_append: base/scale must be positive and finite, proportion in [0,1]");
    const aionhip_weight *ws[3] = {wq, wk, wv};
    for (const aionhip_weight *w : ws)
        if (w->k != wq->k || w->dtype != wq->dtype) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "qkv_rope_append: weights must share k and dtype");
    if (wq->dtype == AIONHIP_F32) return set_err(ctx, AIONHIP_UNSUPPORTED, "qkv_rope_append: f32 weights run as single MatMulNT steps");
    if (d == 0 || d % 8 != 0 || d > 65528 || h_q == 0 || h_kv == 0 || wq->n != h_q * d || wk->n != h_kv * d || wv->n != h_kv * d)
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "qkv_rope_append: weight rows must be heads x head size, head size a multiple of 8");
    // one token of one sequence, short enough K for the in-kernel prologue: anything else takes the separate steps
    if (wq->k > FUSED_MAX_K || ((x | gamma | beta_norm) & 15) || (q_out & 3) || ((k_cache | v_cache) & 1) || t_cap == 0 || t_cap > 0x7FFFFFFFu)
        return set_err(ctx, AIONHIP_UNSUPPORTED, "qkv_rope_append: needs k <= %zu, 16-byte aligned x/gamma/beta and a cache of 1..2^31-1 tokens", FUSED_MAX_K);
    const size_t half = d / 2;
    size_t rope_pairs = (size_t)floorf(rope_proportion * (float)half);
    if (rope_pairs > half) rope_pairs = half;
    const float freq_step = (float)pow((double)base_frequency, (double)(-2.0f / (float)d));
    const float *freq = nullptr;
    int rc = rope_table(ctx, (int)rope_pairs, freq_step, scale_factor, &freq);
    if (rc) return rc;
    FusedEpi epi{(const int *)(uintptr_t)positions, (const int *)(uintptr_t)write_index, freq, (__half *)(uintptr_t)k_cache,
                 (__half *)(uintptr_t)v_cache, (int)t_cap, (int)h_kv, (int)d, (int)rope_pairs, rolling ? 1 : 0};
    FusedIn in{(const float *)(uintptr_t)x, nullptr, (const float *)(uintptr_t)gamma, (const float *)(uintptr_t)beta_norm, eps};
    return launch_gemv_fused_rope(ctx, ws, (float *)(uintptr_t)q_out, in, epi);
}

int aionhip_step_rmsnorm_geglu_matmul(aionhip_ctx *ctx, const aionhip_weight *w_gate, const aionhip_weight *w_up, const aionhip_weight *w_down,
                                      aionhip_handle x, aionhip_handle gamma, aionhip_handle beta_norm, float eps,
                                      aionhip_handle c, float alpha, float beta) {
    if (!ctx || !w_gate || !w_up || !w_down) return AIONHIP_INVALID_ARGUMENT;
    if (!x || !gamma || !c) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "geglu_matmul: null operand");
    if (!(eps > 0.f) || !(eps < INFINITY)) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "geglu_matmul: eps must be positive and finite");
    if (w_gate->k != w_up->k || w_gate->n != w_up->n || w_gate->dtype != w_up->dtype || w_down->k != w_gate->n)
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "geglu_matmul: gate and up must match, down must take their outputs");
    if (w_gate->dtype == AIONHIP_F32 || w_down->dtype == AIONHIP_F32) return set_err(ctx, AIONHIP_UNSUPPORTED, "geglu_matmul: f32 weights run as single MatMulNT steps");
    if (c & 3) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "geglu_matmul: C not 4-byte aligned");
    if (w_gate->k > FUSED_MAX_K || w_gate->n % 32 != 0 || ((x | gamma | beta_norm) & 15))
        return set_err(ctx, AIONHIP_UNSUPPORTED, "geglu_matmul: needs k <= %zu, a hidden size that is a multiple of 32 and 16-byte aligned x/gamma/beta", FUSED_MAX_K);
    int rc = ensure_scratch(ctx, prepared_act_bytes(1, w_down->k));
    if (rc) return rc;
    PreparedAct act = prepared_act_carve(ctx->scratch, 1, w_down->k);
    FusedIn in{(const float *)(uintptr_t)x, nullptr, (const float *)(uintptr_t)gamma, (const float *)(uintptr_t)beta_norm, eps};
    rc = launch_gemv_fused_geglu(ctx, w_gate, w_up, in, act);
    if (rc) return rc;
    float *cp = (float *)(uintptr_t)c;
    const size_t ldc = w_down->n;
    return launch_gemv_batch(ctx, &w_down, &cp, &ldc, 1, 1, act, alpha, beta);
}

int aionhip_step_gate_matmul(aionhip_ctx *ctx, const aionhip_weight *w, size_t rows, aionhip_handle gate, aionhip_handle up,
                             aionhip_handle c, size_t ldc, float alpha, float beta) {
    if (!ctx || !w) return AIONHIP_INVALID_ARGUMENT;
    if (rows == 0) return AIONHIP_OK;
    Batch b;
    int rc = check_batch(ctx, "gate_matmul", 1, &w, &c, &ldc, b);
    if (rc) return rc;
    if (!gate || !up || ((gate | up) & 3)) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "gate_matmul: null or misaligned gate/up");
    const float *gp = (const float *)(uintptr_t)gate, *up_p = (const float *)(uintptr_t)up;
    if (rows == 1 && fused_row_pays(b) && ((gate | up) & 15) == 0)
        return launch_gemv_fused(ctx, b.w, b.c, b.ldc, 1, PRO_GATE, FusedIn{gp, up_p, nullptr, nullptr, 0.f}, alpha, beta);
    // more rows, on the exact kernels (always, or where the bf16 kernel would not pay): the same two launches, the GEMM last
    const bool bf16_route = rows > GEMV_MAX_M && (ctx->gemm_mode == AIONHIP_GEMM_BF16_MFMA_ALWAYS ||
                                                  (ctx->gemm_mode == AIONHIP_GEMM_BF16_MFMA && gemm_bf16_pays(ctx, rows, b.w[0]->n, b.k)));
    if (!bf16_route && rows <= 0x7FFFFFFFu) {
        // gate and activation preparation in one small launch, then the GEMV (or GEMM) on the prepared rows
        rc = ensure_scratch(ctx, prepared_act_bytes(rows, b.k));
        if (rc) return rc;
        PreparedAct act = prepared_act_carve(ctx->scratch, rows, b.k);
        rc = launch_prepare_gate(ctx, gp, up_p, rows, b.k, act);
        if (rc) return rc;
        return launch_prepared_rows(ctx, b, rows, act, alpha, beta);
    }
    const size_t act_bytes = (prepared_act_bytes(rows, b.k) + 255) & ~(size_t)255;
    rc = ensure_scratch(ctx, act_bytes + rows * b.k * sizeof(float));
    if (rc) return rc;
    float *h = (float *)((char *)ctx->scratch + act_bytes);
    rc = launch_gate_gelu(ctx, h, gp, up_p, rows * b.k);
    if (rc) return rc;
    return run_rows(ctx, b, rows, h, b.k, alpha, beta);
}

}  // extern "C"
