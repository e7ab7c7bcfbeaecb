// Decode GEMV: C[b, n] = alpha * sum_kb (a_scale[b,kb] * w_scale[n,kb]) * idot(aq[b,kb], wq[n,kb]) + beta*C
// for 1..8 activation rows against a q8_0 or q4_0 weight in the device row layout.
//
// Arithmetic is aion's CPU decode path (cpu/kernels/matmul_nt_q.zig:74-95,
// cpu/kernels/matvec_q.zig:118-160, cpu/kernels/matmul_q_i8.zig:436-470): exact int8 block
// dots, f32 scale-accumulate. Only the f32 summation order differs (lanes own K slices here).
//
// Mapping: one wavefront owns R consecutive weight rows. Lane l streams 16-byte chunks
// l, l+64, ... of each row (q8: 16 codes = half a block; q4: 32 nibbles = one block), so a
// wavefront load instruction covers 1 KiB of contiguous HBM. The B activation rows' chunks
// are loaded once per iteration and reused for the R rows. Partial sums are folded across the
// wavefront with DPP + two permutes. HBM-bound: algorithmic bytes = N*K/32*{34|18}.
#include "common.h"

namespace {

template <int DT, int B, int R>
__global__ __launch_bounds__(256) void gemv_kernel(GemvBatch batch, const u32x4 *__restrict__ aq, const float *__restrict__ a_scale,
                                                   const int *__restrict__ a_sum, int K, int m, float alpha, float beta) {
    const int lane = threadIdx.x & 63;
    const int gwave = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // uniform: keep it scalar
    if (gwave >= batch.total_waves) return;
    int si = 0;
#pragma unroll
    for (int i = 1; i < 4; ++i)
        if (i < batch.count && gwave >= batch.seg[i].first_wave) si = i;
    const u32x4 *__restrict__ qs = batch.seg[si].qs;
    const __half *__restrict__ sc = batch.seg[si].sc;
    float *__restrict__ c = batch.seg[si].c;
    const size_t ldc = batch.seg[si].ldc;
    const int N = batch.seg[si].n;
    const int row0 = (gwave - batch.seg[si].first_wave) * R;
    const int KB = K >> 5;
    constexpr bool Q8 = DT == AIONHIP_Q8_0;
    const int chunks = Q8 ? (K >> 4) : KB;      // 16-byte weight chunks per row
    const int a_chunks = K >> 4;                // 16-byte activation chunks per row

    float acc[R][B];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int b = 0; b < B; ++b) acc[r][b] = 0.f;

    size_t rowq[R], rows[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int row = min(row0 + r, N - 1);
        rowq[r] = (size_t)row * chunks;
        rows[r] = (size_t)row * KB;
    }

#pragma unroll 2
    for (int ch = lane; ch < chunks; ch += 64) {
        const int blk = Q8 ? (ch >> 1) : ch;
        u32x4 w[R];
        float ws[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            w[r] = __builtin_nontemporal_load(qs + rowq[r] + ch);
            ws[r] = __half2float(sc[rows[r] + blk]);
        }
#pragma unroll
        for (int b = 0; b < B; ++b) {
            const int br = min(b, m - 1);
            const float as = a_scale[(size_t)br * KB + blk];
            if (Q8) {
                const u32x4 a = aq[(size_t)br * a_chunks + ch];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    int d = dot4_i8((int)a.x, (int)w[r].x, 0);
                    d = dot4_i8((int)a.y, (int)w[r].y, d);
                    d = dot4_i8((int)a.z, (int)w[r].z, d);
                    d = dot4_i8((int)a.w, (int)w[r].w, d);
                    acc[r][b] += (float)d * (as * ws[r]);
                }
            } else {
                const u32x4 a0 = aq[(size_t)br * a_chunks + 2 * ch];
                const u32x4 a1 = aq[(size_t)br * a_chunks + 2 * ch + 1];
                const int bias = 8 * a_sum[(size_t)br * KB + blk];   // codes are nibble-8
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    constexpr unsigned M = 0x0F0F0F0Fu;
                    int d = dot4_i8((int)a0.x, (int)(w[r].x & M), -bias);
                    d = dot4_i8((int)a0.y, (int)((w[r].x >> 4) & M), d);
                    d = dot4_i8((int)a0.z, (int)(w[r].y & M), d);
                    d = dot4_i8((int)a0.w, (int)((w[r].y >> 4) & M), d);
                    d = dot4_i8((int)a1.x, (int)(w[r].z & M), d);
                    d = dot4_i8((int)a1.y, (int)((w[r].z >> 4) & M), d);
                    d = dot4_i8((int)a1.z, (int)(w[r].w & M), d);
                    d = dot4_i8((int)a1.w, (int)((w[r].w >> 4) & M), d);
                    acc[r][b] += (float)d * (as * ws[r]);
                }
            }
        }
    }

#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int b = 0; b < B; ++b) acc[r][b] = wave_sum(acc[r][b]);

    if (lane == 0) {
#pragma unroll
        for (int b = 0; b < B; ++b) {
            if (b >= m) break;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (row0 + r >= N) break;
                float *dst = c + (size_t)b * ldc + row0 + r;
                const float v = alpha * acc[r][b];
                *dst = beta == 0.f ? v : v + beta * *dst;
            }
        }
    }
}

template <int DT, int B>
void launch_r(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, int m,
              PreparedAct act, float alpha, float beta) {
    const int K = (int)ws[0]->k;
    long n_total = 0;
    for (int i = 0; i < count; ++i) n_total += (long)ws[i]->n;
    // rows per wavefront: enough wavefronts to give every CU ~8, then amortise activation loads
    const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
    int R = 4;
    if (n_total < (long)cus * 8 * 4) R = 2;
    if (n_total < (long)cus * 8 * 2) R = 1;
    if (B >= 4 && R < 2 && n_total >= cus * 4) R = 2;   // batched rows are VALU-heavy: reuse the activation registers
    GemvBatch batch{};
    batch.count = count;
    int waves = 0;
    for (int i = 0; i < count; ++i) {
        batch.seg[i] = GemvSeg{(const u32x4 *)ws[i]->qs, ws[i]->sc, cs[i], ldcs[i], (int)ws[i]->n, waves};
        waves += ((int)ws[i]->n + R - 1) / R;
    }
    batch.total_waves = waves;
    const auto *aq = (const u32x4 *)act.q;
    const dim3 grid((unsigned)((waves + 3) / 4)), block(256);
    if (R == 4) launch_k(ctx, gemv_kernel<DT, B, 4>, grid, block, 0, batch, aq, act.scale, act.sum, K, m, alpha, beta);
    else if (R == 2) launch_k(ctx, gemv_kernel<DT, B, 2>, grid, block, 0, batch, aq, act.scale, act.sum, K, m, alpha, beta);
    else launch_k(ctx, gemv_kernel<DT, B, 1>, grid, block, 0, batch, aq, act.scale, act.sum, K, m, alpha, beta);
}

template <int DT>
void launch_b(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, int m,
              PreparedAct act, float alpha, float beta) {
    if (m == 1) launch_r<DT, 1>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
    else if (m == 2) launch_r<DT, 2>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
    else if (m <= 4) launch_r<DT, 4>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
    else launch_r<DT, 8>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
}

}  // namespace

int launch_gemv_batch(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, int m,
                      PreparedAct act, float alpha, float beta) {
    if (m < 1 || m > 8) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "gemv: m=%d outside 1..8", m);
    if (count < 1 || count > 4) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "gemv: %d weights in one launch (1..4)", count);
    const char *name = ws[0]->dtype == AIONHIP_Q8_0 ? "gemv_q8" : "gemv_q4";
    ProfScope scope(ctx, name);
    if (ws[0]->dtype == AIONHIP_Q8_0) launch_b<AIONHIP_Q8_0>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
    else launch_b<AIONHIP_Q4_0>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
    LAUNCH_CHECK(ctx, name);
    return AIONHIP_OK;
}

int launch_gemv(aionhip_ctx *ctx, const aionhip_weight *w, int m, PreparedAct act, float *c, size_t ldc, float alpha, float beta) {
    return launch_gemv_batch(ctx, &w, &c, &ldc, 1, m, act, alpha, beta);
}
