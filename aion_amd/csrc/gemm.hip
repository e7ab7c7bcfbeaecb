// Prefill GEMM back ends (m > 8 activation rows).
#include "common.h"

int launch_gemm_i8(aionhip_ctx *ctx, const aionhip_weight *w, size_t m, PreparedAct act, float *c, size_t ldc, float alpha, float beta) {
    // first correct path: row panels of 8 through the decode kernel (re-streams W per panel)
    const size_t KB = w->k / QK;
    for (size_t r0 = 0; r0 < m; r0 += 8) {
        const int mm = (int)(m - r0 < 8 ? m - r0 : 8);
        PreparedAct sub{act.q + r0 * w->k, act.scale + r0 * KB, act.sum + r0 * KB};
        int rc = launch_gemv(ctx, w, mm, sub, c + r0 * ldc, ldc, alpha, beta);
        if (rc) return rc;
    }
    ctx->last_kernel = w->dtype == AIONHIP_Q8_0 ? "gemm_i8_panels_q8" : "gemm_i8_panels_q4";
    return AIONHIP_OK;
}

int launch_gemm_bf16(aionhip_ctx *ctx, const aionhip_weight *, size_t, const float *, size_t, float *, size_t, float, float) {
    return set_err(ctx, AIONHIP_UNSUPPORTED, "bf16 MFMA GEMM is not built yet");
}
