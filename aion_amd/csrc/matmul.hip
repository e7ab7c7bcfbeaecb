// StepMatMul / StepMatMulNT entry points: argument checks (the aion compiler's validation,
// graph/program/compiler.zig:189-239,337-357), activation preparation, kernel routing
// (the counterpart of cpu/exec/matmul.zig:233-296 `matvecRoute` / `gemm2D`).
#include "common.h"

namespace {

constexpr size_t GEMV_MAX_M = 8;

int run_matmul(aionhip_ctx *ctx, const aionhip_weight *b, size_t m, aionhip_handle a_h, size_t lda,
               aionhip_handle c_h, size_t ldc, float alpha, float beta) {
    if (m == 0) return AIONHIP_OK;
    if (!a_h || !c_h) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "matmul: null A or C");
    if (lda == 0) lda = b->k;
    if (ldc == 0) ldc = b->n;
    if (lda < b->k || ldc < b->n) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "matmul: lda=%zu < k=%zu or ldc=%zu < n=%zu", lda, b->k, ldc, b->n);
    if ((a_h & 3) || (c_h & 3)) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "matmul: A and C must be 4-byte aligned");
    if (m > 0x7FFFFFFFu) return set_err(ctx, AIONHIP_UNSUPPORTED, "matmul: m exceeds 2^31-1");
    const float *a = (const float *)(uintptr_t)a_h;
    float *c = (float *)(uintptr_t)c_h;

    if (m > GEMV_MAX_M && ctx->gemm_mode == AIONHIP_GEMM_BF16_MFMA)
        return launch_gemm_bf16(ctx, b, m, a, lda, c, ldc, alpha, beta);

    int rc = ensure_scratch(ctx, prepared_act_bytes(m, b->k));
    if (rc) return rc;
    PreparedAct act = prepared_act_carve(ctx->scratch, m, b->k);
    rc = launch_prepare_act(ctx, a, lda, m, b->k, act);
    if (rc) return rc;
    if (m <= GEMV_MAX_M) return launch_gemv(ctx, b, (int)m, act, c, ldc, alpha, beta);
    return launch_gemm_i8(ctx, b, m, act, c, ldc, alpha, beta);
}

int run_matmul_batch(aionhip_ctx *ctx, size_t count, const aionhip_weight *const *bs, size_t m, aionhip_handle a_h, size_t lda,
                     const aionhip_handle *c_hs, const size_t *ldcs_in, float alpha, float beta) {
    if (count == 0 || m == 0) return AIONHIP_OK;
    if (count > 4) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "matmul_batch: at most 4 weights per call");
    if (!bs || !c_hs || !a_h) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "matmul_batch: null argument");
    const size_t k = bs[0] ? bs[0]->k : 0;
    float *cs[4];
    size_t ldcs[4];
    for (size_t i = 0; i < count; ++i) {
        if (!bs[i] || !c_hs[i]) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "matmul_batch: null weight or C");
        if (bs[i]->k != k || bs[i]->dtype != bs[0]->dtype) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "matmul_batch: weights must share k and dtype");
        ldcs[i] = ldcs_in && ldcs_in[i] ? ldcs_in[i] : bs[i]->n;
        if (ldcs[i] < bs[i]->n || (c_hs[i] & 3)) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "matmul_batch: bad ldc or C alignment");
        cs[i] = (float *)(uintptr_t)c_hs[i];
    }
    if (lda == 0) lda = k;
    if (lda < k || (a_h & 3)) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "matmul_batch: bad lda or A alignment");
    if (m > GEMV_MAX_M) {
        // prefill: the weights run one after the other (each is MFMA-bound on its own)
        for (size_t i = 0; i < count; ++i) {
            int rc = run_matmul(ctx, bs[i], m, a_h, lda, c_hs[i], ldcs[i], alpha, beta);
            if (rc) return rc;
        }
        return AIONHIP_OK;
    }
    int rc = ensure_scratch(ctx, prepared_act_bytes(m, k));
    if (rc) return rc;
    PreparedAct act = prepared_act_carve(ctx->scratch, m, k);
    rc = launch_prepare_act(ctx, (const float *)(uintptr_t)a_h, lda, m, k, act);
    if (rc) return rc;
    return launch_gemv_batch(ctx, bs, cs, ldcs, (int)count, (int)m, act, alpha, beta);
}

}  // namespace

extern "C" {

int aionhip_step_matmul_batch(aionhip_ctx *ctx, size_t count, const aionhip_weight *const *b, size_t m, aionhip_handle a, size_t lda,
                              const aionhip_handle *c, const size_t *ldc, float alpha, float beta) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    return run_matmul_batch(ctx, count, b, m, a, lda, c, ldc, alpha, beta);
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
    // StepMatMulNT: B is q8_0 [N,K] with quant_axis 1 (runtime/executable.zig:211-223)
    if (b->layout != AIONHIP_ROWS_NK || b->dtype != AIONHIP_Q8_0) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "MatMulNT needs a q8_0 [N,K] weight (quant_axis 1)");
    return run_matmul(ctx, b, m, a, lda, c, ldc, alpha, beta);
}

}  // extern "C"
