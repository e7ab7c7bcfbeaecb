// Per-token glue steps (placeholder until the kernels land): every call is rejected loudly.
#include "common.h"

extern "C" {
int aionhip_step_rmsnorm(aionhip_ctx *ctx, aionhip_handle, aionhip_handle, aionhip_handle, aionhip_handle, aionhip_handle, size_t, size_t, float) { return set_err(ctx, AIONHIP_UNSUPPORTED, "rmsnorm is not built yet"); }
int aionhip_step_rope(aionhip_ctx *ctx, aionhip_handle, aionhip_handle, aionhip_handle, size_t, size_t, size_t, size_t, float, float, float) { return set_err(ctx, AIONHIP_UNSUPPORTED, "rope is not built yet"); }
int aionhip_step_add(aionhip_ctx *ctx, aionhip_handle, aionhip_handle, aionhip_handle, size_t) { return set_err(ctx, AIONHIP_UNSUPPORTED, "add is not built yet"); }
int aionhip_step_gate_gelu(aionhip_ctx *ctx, aionhip_handle, aionhip_handle, aionhip_handle, size_t) { return set_err(ctx, AIONHIP_UNSUPPORTED, "gate is not built yet"); }
int aionhip_step_gather_rows(aionhip_ctx *ctx, int, aionhip_handle, aionhip_handle, aionhip_handle, size_t, size_t, size_t) { return set_err(ctx, AIONHIP_UNSUPPORTED, "gather is not built yet"); }
int aionhip_step_append_f16(aionhip_ctx *ctx, aionhip_handle, aionhip_handle, aionhip_handle, size_t, size_t, size_t, size_t) { return set_err(ctx, AIONHIP_UNSUPPORTED, "append is not built yet"); }
int aionhip_step_cast_f32_f16(aionhip_ctx *ctx, aionhip_handle, aionhip_handle, size_t) { return set_err(ctx, AIONHIP_UNSUPPORTED, "cast is not built yet"); }
int aionhip_step_argmax(aionhip_ctx *ctx, aionhip_handle, aionhip_handle, size_t, size_t) { return set_err(ctx, AIONHIP_UNSUPPORTED, "argmax is not built yet"); }
}
