// Attention step (placeholder until the kernels land): rejects every call loudly.
#include "common.h"

extern "C" int aionhip_step_attention(aionhip_ctx *ctx, const aionhip_attention *p) {
    if (!ctx || !p) return AIONHIP_INVALID_ARGUMENT;
    return set_err(ctx, AIONHIP_UNSUPPORTED, "attention is not built yet");
}
