// MatMulNT with an f32 B operand (aion runtime/executable.zig:211-223; cpu/exec/matmul_nt.zig:87-259, kernel
// cpu/kernels/matmul_nt.zig:40-126): C[m, n] = alpha * sum_k A[m, k] * B[n, k] + beta * C[m, n], all f32, no quantization
// anywhere. Off the quantized hot path - a package whose head or projection is kept in f32 - so the kernel is a plain
// streaming one: a wavefront owns one row of B at a time and up to eight rows of A (the rows of A are re-read from cache by
// every wavefront, the row of B comes from memory once per eight rows of A), f32 fused multiply-adds into one partial sum
// per lane and row of A, folded over the wavefront at the end. The summation order differs from aion's (four SIMD
// accumulators over K, cpu/kernels/matmul_nt.zig:68-98); the terms and the f32 arithmetic are the same.
#include "common.h"

namespace {

template <int B, bool VEC>
__global__ __launch_bounds__(256) void matmul_nt_f32_kernel(float *__restrict__ c, const float *__restrict__ a, const float *__restrict__ w, int m0, int m,
                                                            int n, int k, size_t lda, size_t ldc, float alpha, float beta) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n) return;
    const float *__restrict__ wr = w + (size_t)row * k;
    float acc[B];
#pragma unroll
    for (int b = 0; b < B; ++b) acc[b] = 0.f;
    if (VEC) {
        const int k4 = k >> 2;
        for (int i = lane; i < k4; i += 64) {
            const f32x4 wv = __builtin_nontemporal_load((const f32x4 *)wr + i);
#pragma unroll
            for (int b = 0; b < B; ++b) {
                const f32x4 av = *((const f32x4 *)(a + (size_t)min(m0 + b, m - 1) * lda) + i);
                acc[b] = fmaf(av.x, wv.x, acc[b]);
                acc[b] = fmaf(av.y, wv.y, acc[b]);
                acc[b] = fmaf(av.z, wv.z, acc[b]);
                acc[b] = fmaf(av.w, wv.w, acc[b]);
            }
        }
    } else {
        for (int i = lane; i < k; i += 64) {
            const float wv = wr[i];
#pragma unroll
            for (int b = 0; b < B; ++b) acc[b] = fmaf(a[(size_t)min(m0 + b, m - 1) * lda + i], wv, acc[b]);
        }
    }
#pragma unroll
    for (int b = 0; b < B; ++b) acc[b] = wave_sum(acc[b]);
    if (lane == 0) {
#pragma unroll
        for (int b = 0; b < B; ++b) {
            if (m0 + b >= m) break;
            float *dst = c + (size_t)(m0 + b) * ldc + row;
            const float v = alpha * acc[b];
            *dst = beta == 0.f ? v : v + beta * *dst;
        }
    }
}

}  // namespace

int launch_matmul_nt_f32(aionhip_ctx *ctx, const aionhip_weight *w, size_t m, const float *a, size_t lda, float *c, size_t ldc, float alpha,
                         float beta) {
    ProfScope scope(ctx, "matmul_nt_f32");
    const int n = (int)w->n, k = (int)w->k;
    const bool vec = (k & 3) == 0 && (lda & 3) == 0 && ((uintptr_t)a & 15) == 0;
    const dim3 grid((unsigned)((n + 3) / 4)), block(256);
    const float *wd = (const float *)w->qs;
    for (size_t m0 = 0; m0 < m; m0 += 8) {
        const size_t left = m - m0;
        if (left == 1) {
            if (vec) launch_k(ctx, matmul_nt_f32_kernel<1, true>, grid, block, 0, c, a, wd, (int)m0, (int)m, n, k, lda, ldc, alpha, beta);
            else launch_k(ctx, matmul_nt_f32_kernel<1, false>, grid, block, 0, c, a, wd, (int)m0, (int)m, n, k, lda, ldc, alpha, beta);
        } else if (left <= 4) {
            if (vec) launch_k(ctx, matmul_nt_f32_kernel<4, true>, grid, block, 0, c, a, wd, (int)m0, (int)m, n, k, lda, ldc, alpha, beta);
            else launch_k(ctx, matmul_nt_f32_kernel<4, false>, grid, block, 0, c, a, wd, (int)m0, (int)m, n, k, lda, ldc, alpha, beta);
        } else {
            if (vec) launch_k(ctx, matmul_nt_f32_kernel<8, true>, grid, block, 0, c, a, wd, (int)m0, (int)m, n, k, lda, ldc, alpha, beta);
            else launch_k(ctx, matmul_nt_f32_kernel<8, false>, grid, block, 0, c, a, wd, (int)m0, (int)m, n, k, lda, ldc, alpha, beta);
        }
    }
    LAUNCH_CHECK(ctx, "matmul_nt_f32");
    return AIONHIP_OK;
}
