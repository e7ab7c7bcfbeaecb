// Weight ingest: aion's packed q8_0/q4_0 blocks -> the device-private row layout the kernels
// stream (see aionhip_weight in common.h). A pure byte permutation: nothing is requantized,
// and aionhip_weight_download inverts it byte-exactly (the property aion's own re-lay pass is
// tested for, graph/opt/test_opt.zig:921-959).
#include "common.h"

#include <new>

namespace {

__device__ __forceinline__ unsigned load_u16(const uint8_t *p) { return *reinterpret_cast<const uint16_t *>(p); }

// thread i handles block i of the SOURCE order, so reads are coalesced; src block index ->
// (n, kb): ROWS_NK: i = n*KB + kb; KMAJOR: i = kb*ld + n (n < N).
template <int DT, bool KMAJOR, bool INVERSE>
__global__ void relay_kernel(uint8_t *__restrict__ packed, uint8_t *__restrict__ qs, __half *__restrict__ sc,
                             size_t N, size_t KB, size_t ld) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t n, kb;
    if (KMAJOR) {
        if (i >= KB * N) return;
        kb = i / N;
        n = i % N;
    } else {
        if (i >= N * KB) return;
        n = i / KB;
        kb = i % KB;
    }
    constexpr int BB = DT == AIONHIP_Q8_0 ? Q8_BYTES : Q4_BYTES;
    uint8_t *blk = packed + (KMAJOR ? (kb * ld + n) : (n * KB + kb)) * BB;
    uint16_t *s16 = reinterpret_cast<uint16_t *>(sc) + n * KB + kb;
    if (DT == AIONHIP_Q8_0) {
        uint32_t *q = reinterpret_cast<uint32_t *>(qs + (n * KB + kb) * 32);
        if (!INVERSE) {
            *s16 = (uint16_t)load_u16(blk);
#pragma unroll
            for (int j = 0; j < 8; ++j) q[j] = load_u16(blk + 2 + 4 * j) | (load_u16(blk + 4 + 4 * j) << 16);
        } else {
            *reinterpret_cast<uint16_t *>(blk) = *s16;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t w = q[j];
                *reinterpret_cast<uint16_t *>(blk + 2 + 4 * j) = (uint16_t)w;
                *reinterpret_cast<uint16_t *>(blk + 4 + 4 * j) = (uint16_t)(w >> 16);
            }
        }
    } else {
        // source byte b holds element 2b (low nibble) and 2b+1 (high nibble). Word j covers
        // elements 8j..8j+7 = source bytes 4j..4j+3; target byte i = e[8j+i] | e[8j+4+i] << 4.
        uint32_t *q = reinterpret_cast<uint32_t *>(qs + (n * KB + kb) * 16);
        if (!INVERSE) {
            *s16 = (uint16_t)load_u16(blk);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t s = load_u16(blk + 2 + 4 * j) | (load_u16(blk + 4 + 4 * j) << 16);
                uint32_t e[8];
#pragma unroll
                for (int t = 0; t < 8; ++t) e[t] = (s >> (4 * t)) & 15u;
                uint32_t w = 0;
#pragma unroll
                for (int b = 0; b < 4; ++b) w |= (e[b] | (e[4 + b] << 4)) << (8 * b);
                q[j] = w;
            }
        } else {
            *reinterpret_cast<uint16_t *>(blk) = *s16;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t w = q[j];
                uint32_t s = 0;
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const uint32_t byte = (w >> (8 * b)) & 0xFFu;
                    s |= (byte & 15u) << (4 * b);         // element b
                    s |= (byte >> 4) << (4 * (4 + b));    // element 4+b
                }
                *reinterpret_cast<uint16_t *>(blk + 2 + 4 * j) = (uint16_t)s;
                *reinterpret_cast<uint16_t *>(blk + 4 + 4 * j) = (uint16_t)(s >> 16);
            }
        }
    }
}

template <bool INVERSE>
int run_relay(aionhip_ctx *ctx, const aionhip_weight *w, uint8_t *packed, size_t ld) {
    const size_t KB = w->k / QK;
    const size_t total = w->n * KB;
    if (!total) return AIONHIP_OK;
    const dim3 grid((unsigned)((total + 255) / 256)), block(256);
    const bool km = w->layout == AIONHIP_KMAJOR_KN;
    if (w->dtype == AIONHIP_Q8_0) {
        if (km) relay_kernel<AIONHIP_Q8_0, true, INVERSE><<<grid, block, 0, ctx->stream>>>(packed, w->qs, w->sc, w->n, KB, ld);
        else relay_kernel<AIONHIP_Q8_0, false, INVERSE><<<grid, block, 0, ctx->stream>>>(packed, w->qs, w->sc, w->n, KB, ld);
    } else {
        if (km) relay_kernel<AIONHIP_Q4_0, true, INVERSE><<<grid, block, 0, ctx->stream>>>(packed, w->qs, w->sc, w->n, KB, ld);
        else relay_kernel<AIONHIP_Q4_0, false, INVERSE><<<grid, block, 0, ctx->stream>>>(packed, w->qs, w->sc, w->n, KB, ld);
    }
    LAUNCH_CHECK(ctx, "weight_relay");
    return AIONHIP_OK;
}

int check_weight_args(aionhip_ctx *ctx, int dtype, int layout, size_t n, size_t k, size_t ld) {
    if (dtype == AIONHIP_F32) {
        // the f32 operand of MatMulNT (runtime/executable.zig:211-223, cpu/exec/matmul_nt.zig:100): rows [N,K] as they are
        if (layout != AIONHIP_ROWS_NK) return set_err(ctx, AIONHIP_UNSUPPORTED, "f32 weights are the [N,K] operand of MatMulNT only");
        if (n == 0 || k == 0) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "weight shape n=%zu k=%zu", n, k);
        if (n > 0x7FFFFFFFu || k > 0x7FFFFFFFu) return set_err(ctx, AIONHIP_UNSUPPORTED, "weight dimension exceeds 2^31-1");
        if (ld != 0) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "ld_blocks applies to K-major quantized weights");
        return AIONHIP_OK;
    }
    if (dtype != AIONHIP_Q8_0 && dtype != AIONHIP_Q4_0) return set_err(ctx, AIONHIP_UNSUPPORTED, "weight dtype %d is not q8_0 / q4_0 / f32", dtype);
    if (layout != AIONHIP_ROWS_NK && layout != AIONHIP_KMAJOR_KN) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "unknown weight layout %d", layout);
    // aion has no q4 [N,K] operand (cpu/exec/matmul.zig:233-239): MatMulNT is q8 or f32 only
    if (dtype == AIONHIP_Q4_0 && layout == AIONHIP_ROWS_NK) return set_err(ctx, AIONHIP_UNSUPPORTED, "q4_0 weights are K-major [K,N] only");
    if (n == 0 || k == 0 || k % QK != 0) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "weight shape n=%zu k=%zu: k must be a positive multiple of 32", n, k);
    if (n > 0x7FFFFFFFu || k > 0x7FFFFFFFu) return set_err(ctx, AIONHIP_UNSUPPORTED, "weight dimension exceeds 2^31-1");
    if (ld != 0 && (layout != AIONHIP_KMAJOR_KN || ld < n)) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "ld_blocks %zu invalid for n=%zu", ld, n);
    return AIONHIP_OK;
}

int alloc_weight(aionhip_ctx *ctx, int dtype, int layout, size_t n, size_t k, aionhip_weight **out) {
    aionhip_weight *w = new (std::nothrow) aionhip_weight();
    if (!w) return set_err(ctx, AIONHIP_OUT_OF_MEMORY, "host allocation failed");
    w->dtype = dtype;
    w->layout = layout;
    w->n = n;
    w->k = k;
    w->qs_bytes = dtype == AIONHIP_F32 ? n * k * sizeof(float) : (dtype == AIONHIP_Q8_0 ? n * k : n * k / 2);
    w->sc_bytes = dtype == AIONHIP_F32 ? 0 : n * (k / QK) * sizeof(__half);
    // one allocation: quants first (16-byte aligned rows since k % 32 == 0), scales after
    const size_t qs_padded = (w->qs_bytes + 255) & ~(size_t)255;
    void *p = nullptr;
    const int rc = dev_malloc(ctx, &p, qs_padded + w->sc_bytes + 256, "a weight");  // slack: kernels may read one 16-byte chunk of a clamped row
    if (rc) {
        delete w;
        return rc;
    }
    w->qs = (uint8_t *)p;
    w->sc = (__half *)((uint8_t *)p + qs_padded);
    *out = w;
    return AIONHIP_OK;
}

}  // namespace

extern "C" {

int aionhip_weight_from_device(aionhip_ctx *ctx, int dtype, int layout, size_t n, size_t k, size_t ld_blocks,
                               aionhip_handle device_blocks, aionhip_weight **out) {
    if (!ctx || !out || !device_blocks) return AIONHIP_INVALID_ARGUMENT;
    *out = nullptr;
    int rc = check_weight_args(ctx, dtype, layout, n, k, ld_blocks);
    if (rc) return rc;
    aionhip_weight *w = nullptr;
    rc = alloc_weight(ctx, dtype, layout, n, k, &w);
    if (rc) return rc;
    if (dtype == AIONHIP_F32) {
        const hipError_t e = hipMemcpyAsync(w->qs, (const void *)(uintptr_t)device_blocks, w->qs_bytes, hipMemcpyDeviceToDevice, ctx->stream);
        rc = e == hipSuccess ? (int)AIONHIP_OK : set_err(ctx, AIONHIP_EXECUTION_FAILED, "f32 weight copy: %s", hipGetErrorString(e));
    } else {
        rc = run_relay<false>(ctx, w, (uint8_t *)(uintptr_t)device_blocks, ld_blocks ? ld_blocks : n);
    }
    if (rc) {
        aionhip_weight_free(ctx, w);
        return rc;
    }
    *out = w;
    return AIONHIP_OK;
}

int aionhip_weight_upload(aionhip_ctx *ctx, int dtype, int layout, size_t n, size_t k, size_t ld_blocks,
                          const void *host_blocks, aionhip_weight **out) {
    if (!ctx || !out || !host_blocks) return AIONHIP_INVALID_ARGUMENT;
    *out = nullptr;
    int rc = check_weight_args(ctx, dtype, layout, n, k, ld_blocks);
    if (rc) return rc;
    const size_t bb = dtype == AIONHIP_Q8_0 ? Q8_BYTES : Q4_BYTES;
    const size_t KB = k / QK;
    const size_t ld = ld_blocks ? ld_blocks : n;
    const size_t bytes = dtype == AIONHIP_F32 ? n * k * sizeof(float) : (layout == AIONHIP_KMAJOR_KN ? ((KB - 1) * ld + n) : n * KB) * bb;
    void *staging = nullptr;
    rc = dev_malloc(ctx, &staging, bytes, "weight upload staging");
    if (rc) return rc;
    hipError_t e = hipMemcpyAsync(staging, host_blocks, bytes, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        (void)hipFree(staging);
        return set_err(ctx, AIONHIP_EXECUTION_FAILED, "weight upload copy: %s", hipGetErrorString(e));
    }
    rc = aionhip_weight_from_device(ctx, dtype, layout, n, k, ld_blocks, (aionhip_handle)(uintptr_t)staging, out);
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipFree(staging);
    return rc;
}

// releases this context's bf16 copy of the weight, if it holds one (the caller has waited for the stream)
static void drop_bf16_copy(aionhip_ctx *ctx, const aionhip_weight *w) {
    auto it = ctx->bf16_copies.find(w);
    if (it == ctx->bf16_copies.end()) return;
    (void)hipFree(it->second.first);
    ctx->bf16_copy_bytes -= it->second.second;
    ctx->bf16_copies.erase(it);
}

void aionhip_weight_drop_bf16(aionhip_ctx *ctx, aionhip_weight *w) {
    if (!ctx || !w || ctx->capturing || ctx->bf16_copies.find(w) == ctx->bf16_copies.end()) return;
    (void)hipStreamSynchronize(ctx->stream);      // launches that read the copy may still be queued
    drop_bf16_copy(ctx, w);
}

int aionhip_set_bf16_weight_copies(aionhip_ctx *ctx, int on) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    ctx->bf16_copies_on = on != 0;
    return AIONHIP_OK;
}

int aionhip_bf16_copy_stats(aionhip_ctx *ctx, uint64_t *weights, uint64_t *bytes) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (weights) *weights = (uint64_t)ctx->bf16_copies.size();
    if (bytes) *bytes = (uint64_t)ctx->bf16_copy_bytes;
    return AIONHIP_OK;
}

void aionhip_weight_free(aionhip_ctx *ctx, aionhip_weight *w) {
    if (!w) return;
    if (ctx) (void)hipStreamSynchronize(ctx->stream);
    if (ctx) drop_bf16_copy(ctx, w);
    if (w->qs) (void)hipFree(w->qs);
    delete w;
}

size_t aionhip_weight_packed_bytes(const aionhip_weight *w) {
    if (!w) return 0;
    if (w->dtype == AIONHIP_F32) return w->n * w->k * sizeof(float);
    return w->n * (w->k / QK) * (w->dtype == AIONHIP_Q8_0 ? Q8_BYTES : Q4_BYTES);
}
size_t aionhip_weight_device_bytes(const aionhip_weight *w) { return w ? w->qs_bytes + w->sc_bytes : 0; }

int aionhip_weight_download(aionhip_ctx *ctx, const aionhip_weight *w, void *host_blocks, size_t bytes) {
    if (!ctx || !w || !host_blocks) return AIONHIP_INVALID_ARGUMENT;
    const size_t want = aionhip_weight_packed_bytes(w);
    if (bytes != want) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "download: buffer is %zu bytes, packed form is %zu", bytes, want);
    if (w->dtype == AIONHIP_F32) {           // kept as uploaded
        hipError_t e = hipMemcpyAsync(host_blocks, w->qs, want, hipMemcpyDeviceToHost, ctx->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        return e == hipSuccess ? (int)AIONHIP_OK : set_err(ctx, AIONHIP_EXECUTION_FAILED, "weight download copy: %s", hipGetErrorString(e));
    }
    void *staging = nullptr;
    int rc = dev_malloc(ctx, &staging, want, "weight download staging");
    if (rc) return rc;
    rc = run_relay<true>(ctx, w, (uint8_t *)staging, w->n);
    if (rc == AIONHIP_OK) {
        hipError_t e = hipMemcpyAsync(host_blocks, staging, want, hipMemcpyDeviceToHost, ctx->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess) rc = set_err(ctx, AIONHIP_EXECUTION_FAILED, "weight download copy: %s", hipGetErrorString(e));
    }
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipFree(staging);
    return rc;
}

}  // extern "C"
