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

// ---- 2..8 activation rows: gemv_rows_kernel. The rows' prepared codes, scales and code sums for the K range
// of the launch are copied into LDS once per workgroup; the wavefronts then stride over the weight rows
// (persistent grid, as in the fused one-row kernel) and read every activation operand from LDS.
// Mapping: LPR lanes per weight row (16 where N allows: a wavefront then works on four rows at once), lane j of
// a row's group streams its 16-byte chunks j, j+LPR, ... - 256 contiguous bytes per row per load instruction -
// and keeps one partial sum per activation row. The fold over a row's lanes is then four DPP adds per
// activation row; with a whole wavefront per weight row every (weight row, activation row) pair costs a
// 64-lane fold with two LDS permutes, as much vector work as the dots themselves at K = 2048.
// q4: the two 16-code halves of a block sit in separate LDS planes, so consecutive lanes read consecutive
// 16 bytes of each. K ranges (kb0, kbn in quant blocks) let a long K run as several launches that each fit
// LDS, beta = 1 after the first.
// NT threads per workgroup: 256, or 1024 when the rows' K range needs most of a CU's LDS (one workgroup per CU then, and
// sixteen wavefronts rather than four to keep loads in flight).
constexpr size_t ROWS_LDS_CAP = 72 * 1024, ROWS_LDS_CAP_WIDE = 158 * 1024;
template <int DT, int B, int LPR, int R, int NT = 256>
__global__ __launch_bounds__(NT) void gemv_rows_kernel(GemvBatch batch, const u32x4 *__restrict__ aq, const float *__restrict__ a_scale,
                                                        const int *__restrict__ a_sum, int K, int m, int kb0, int kbn, float alpha, float beta) {
    extern __shared__ __attribute__((aligned(16))) unsigned char s_rows[];
    constexpr bool Q8 = DT == AIONHIP_Q8_0;
    constexpr int RPW = (64 / LPR) * R;                             // weight rows a wavefront works on at once
    const int tid = threadIdx.x, lane = tid & 63;
    const int grp = lane / LPR, lj = lane % LPR;
    const int KB = K >> 5, a_chunks = K >> 4;
    u32x4 *s_a = (u32x4 *)s_rows;                                   // [B][2 * kbn] 16-byte chunks
    float *s_scale = (float *)(s_rows + (size_t)B * kbn * 32);      // [B][kbn]
    int *s_sum = (int *)(s_scale + B * kbn);                        // [B][kbn]
    // the copy is batched: eight 16-byte loads per thread are requested before the first is stored (a loop of
    // load-then-store round trips costs a memory latency per trip, which for a small N is most of the kernel)
    {
        const int per_row = 2 * kbn, total = B * per_row;
        for (int base = 0; base < total; base += NT * 8) {
            u32x4 v[8];
            int dsti[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int idx = min(base + tid + NT * i, total - 1);
                const int b = idx / per_row, c = idx - b * per_row;
                dsti[i] = b * per_row + (Q8 ? c : ((c & 1) ? kbn + (c >> 1) : (c >> 1)));
                v[i] = aq[(size_t)min(b, m - 1) * a_chunks + 2 * kb0 + c];
            }
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (base + tid + NT * i < total) s_a[dsti[i]] = v[i];
        }
        const int total_s = B * kbn;
        for (int base = 0; base < total_s; base += NT * 4) {
            float sv[4];
            int iv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int idx = min(base + tid + NT * i, total_s - 1);
                const int b = idx / kbn, j = idx - b * kbn;
                sv[i] = a_scale[(size_t)min(b, m - 1) * KB + kb0 + j];
                iv[i] = a_sum[(size_t)min(b, m - 1) * KB + kb0 + j];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (base + tid + NT * i < total_s) { s_scale[base + tid + NT * i] = sv[i]; s_sum[base + tid + NT * i] = iv[i]; }
        }
    }
    __syncthreads();

    const int chunks_row = Q8 ? (K >> 4) : KB;      // 16-byte weight chunks per full row
    const int ch0 = Q8 ? 2 * kb0 : kb0, nch = Q8 ? 2 * kbn : kbn;
    const int wave_stride = gridDim.x * (NT / 64);
    for (int gwave = blockIdx.x * (NT / 64) + __builtin_amdgcn_readfirstlane(tid >> 6); gwave < batch.total_waves; gwave += wave_stride) {
        int si = 0;
#pragma unroll
        for (int i = 1; i < 4; ++i)
            if (i < batch.count && gwave >= batch.seg[i].first_wave) si = i;
        const int N = batch.seg[si].n;
        const int row0 = (gwave - batch.seg[si].first_wave) * RPW + grp * R;      // this lane group's R rows
        const u32x4 *__restrict__ wq[R];
        const __half *__restrict__ wsc[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int rowc = min(row0 + r, N - 1);
            wq[r] = batch.seg[si].qs + (size_t)rowc * chunks_row + ch0;
            wsc[r] = batch.seg[si].sc + (size_t)rowc * KB + kb0;
        }
        float acc[R][B];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int b = 0; b < B; ++b) acc[r][b] = 0.f;

        // one chunk position of the R rows: every activation operand is read from LDS once and used R times
        auto consume = [&](int ch, const u32x4 (&w)[R], const float (&ws)[R]) {
            const int blk = Q8 ? (ch >> 1) : ch;
            if (Q8) {
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    const u32x4 a = s_a[b * 2 * kbn + ch];
                    const float as = s_scale[b * kbn + blk];
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        int d = dot4_i8((int)a.x, (int)w[r].x, 0);
                        d = dot4_i8((int)a.y, (int)w[r].y, d);
                        d = dot4_i8((int)a.z, (int)w[r].z, d);
                        d = dot4_i8((int)a.w, (int)w[r].w, d);
                        acc[r][b] += (float)d * (as * ws[r]);
                    }
                }
            } else {
                constexpr unsigned M = 0x0F0F0F0Fu;
                int wn[R][8];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    wn[r][0] = (int)(w[r].x & M); wn[r][1] = (int)((w[r].x >> 4) & M); wn[r][2] = (int)(w[r].y & M); wn[r][3] = (int)((w[r].y >> 4) & M);
                    wn[r][4] = (int)(w[r].z & M); wn[r][5] = (int)((w[r].z >> 4) & M); wn[r][6] = (int)(w[r].w & M); wn[r][7] = (int)((w[r].w >> 4) & M);
                }
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    const u32x4 a0 = s_a[b * 2 * kbn + ch], a1 = s_a[b * 2 * kbn + kbn + ch];
                    const float as = s_scale[b * kbn + blk];
                    const int bias = -8 * s_sum[b * kbn + blk];          // codes are nibble-8
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        int d = dot4_i8((int)a0.x, wn[r][0], bias);
                        d = dot4_i8((int)a0.y, wn[r][1], d);
                        d = dot4_i8((int)a0.z, wn[r][2], d);
                        d = dot4_i8((int)a0.w, wn[r][3], d);
                        d = dot4_i8((int)a1.x, wn[r][4], d);
                        d = dot4_i8((int)a1.y, wn[r][5], d);
                        d = dot4_i8((int)a1.z, wn[r][6], d);
                        d = dot4_i8((int)a1.w, wn[r][7], d);
                        acc[r][b] += (float)d * (as * ws[r]);
                    }
                }
            }
        };
        // U chunk positions in flight (U * R loads) before the first is consumed (requesting the next group
        // ahead of the dots as well was tried: more registers, no gain)
        constexpr int U = R >= 4 ? 1 : (R == 2 ? 2 : 4);
#pragma unroll 1
        for (int c0 = lj; c0 < nch; c0 += LPR * U) {
            u32x4 w[U][R];
            __half hs[U][R];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ch = min(c0 + LPR * u, nch - 1);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    w[u][r] = __builtin_nontemporal_load(wq[r] + ch);
                    hs[u][r] = wsc[r][Q8 ? (ch >> 1) : ch];
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (c0 + LPR * u < nch) {
                    float ws[R];
#pragma unroll
                    for (int r = 0; r < R; ++r) ws[r] = __half2float(hs[u][r]);
                    consume(c0 + LPR * u, w[u], ws);
                }
            }
        }

#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int b = 0; b < B; ++b) {
                float v = acc[r][b];
                v += dpp_f<DPP_QUAD_XOR1>(v);
                v += dpp_f<DPP_QUAD_XOR2>(v);
                v += dpp_f<DPP_ROW_HALF_MIRROR>(v);
                v += dpp_f<DPP_ROW_MIRROR>(v);
                if (LPR >= 32) v += __shfl_xor(v, 16, 64);
                if (LPR >= 64) v += __shfl_xor(v, 32, 64);
                acc[r][b] = v;
            }
        if (lj == 0) {
            float *__restrict__ c = batch.seg[si].c;
            const size_t ldc = batch.seg[si].ldc;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (row0 + r >= N) break;
#pragma unroll
                for (int b = 0; b < B; ++b) {
                    if (b >= m) break;
                    float *dst = c + (size_t)b * ldc + row0 + r;
                    const float v = alpha * acc[r][b];
                    *dst = beta == 0.f ? v : v + beta * *dst;
                }
            }
        }
    }
}

template <int DT, int B>
int launch_rows(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, int m,
                PreparedAct act, float alpha, float beta) {
    const int K = (int)ws[0]->k, KB = K >> 5;
    long n_total = 0;
    for (int i = 0; i < count; ++i) n_total += (long)ws[i]->n;
    const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
    // R rows per lane group: B / 2 at least (an activation operand read from LDS is then used that many times,
    // which keeps the LDS traffic near 5x the weight bytes), fewer only when N is too small for six wavefronts
    // per CU; then the fewest lanes per row (16, 32, 64) that still give six wavefronts per CU
    int R = B >= 8 ? 4 : (B >= 4 ? 2 : 1), lpr = 64;
    while (R > 1 && n_total / R < (long)cus * 6) R >>= 1;
    if (n_total / (R * 4) >= (long)cus * 6) lpr = 16;
    else if (n_total / (R * 2) >= (long)cus * 6) lpr = 32;
    if (lpr == 16 && R < 4 && n_total / (R * 8) >= (long)cus * 6) R *= 2;      // plenty of rows: more reuse per operand
    const int rpw = (64 / lpr) * R;
    GemvBatch batch{};
    batch.count = count;
    int waves = 0;
    for (int i = 0; i < count; ++i) {
        batch.seg[i] = GemvSeg{(const u32x4 *)ws[i]->qs, ws[i]->sc, cs[i], ldcs[i], (int)ws[i]->n, waves};
        waves += ((int)ws[i]->n + rpw - 1) / rpw;
    }
    batch.total_waves = waves;
    // K slices that fit LDS, as even as possible: up to 72 KB per 256-thread workgroup (two or more workgroups per CU); a K
    // that needs more runs in one pass of 1024-thread workgroups with most of the CU's LDS rather than as two launches
    const size_t per_block = (size_t)B * 40;
    const bool wide = (size_t)KB * per_block > ROWS_LDS_CAP && (size_t)KB * per_block <= ROWS_LDS_CAP_WIDE;
    const int max_kbn = (int)((wide ? ROWS_LDS_CAP_WIDE : ROWS_LDS_CAP) / per_block);
    const int slices = (KB + max_kbn - 1) / max_kbn;
    const int kbn_even = (KB + slices - 1) / slices;
    const auto *aq = (const u32x4 *)act.q;
    for (int s = 0, kb0 = 0; s < slices; ++s, kb0 += kbn_even) {
        const int kbn = min(kbn_even, KB - kb0);
        const size_t lds = (size_t)kbn * per_block;
        const int nt = wide ? 1024 : 256;
        const int per_cu = wide ? 1 : (int)min((size_t)8, (size_t)(160 * 1024) / (lds + 512));
        const int wgs = (waves + nt / 64 - 1) / (nt / 64);
        const dim3 grid((unsigned)min(wgs, cus * max(per_cu, 1))), block((unsigned)nt);
        const float b_eff = s == 0 ? beta : 1.f;
        auto go = [&](auto kern) {
            if (lds > 64 * 1024) {
                hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(wide ? ROWS_LDS_CAP_WIDE : ROWS_LDS_CAP));
                if (e != hipSuccess) return set_err(ctx, AIONHIP_EXECUTION_FAILED, "gemv rows: %s", hipGetErrorString(e));
            }
            launch_k(ctx, kern, grid, block, lds, batch, aq, act.scale, act.sum, K, m, kb0, kbn, alpha, b_eff);
            return (int)AIONHIP_OK;
        };
        int rc;
        if (wide) {
            if (R == 4) rc = lpr == 16 ? go(gemv_rows_kernel<DT, B, 16, 4, 1024>) : lpr == 32 ? go(gemv_rows_kernel<DT, B, 32, 4, 1024>) : go(gemv_rows_kernel<DT, B, 64, 4, 1024>);
            else if (R == 2) rc = lpr == 16 ? go(gemv_rows_kernel<DT, B, 16, 2, 1024>) : lpr == 32 ? go(gemv_rows_kernel<DT, B, 32, 2, 1024>) : go(gemv_rows_kernel<DT, B, 64, 2, 1024>);
            else rc = lpr == 16 ? go(gemv_rows_kernel<DT, B, 16, 1, 1024>) : lpr == 32 ? go(gemv_rows_kernel<DT, B, 32, 1, 1024>) : go(gemv_rows_kernel<DT, B, 64, 1, 1024>);
        } else if (R == 4) rc = lpr == 16 ? go(gemv_rows_kernel<DT, B, 16, 4>) : lpr == 32 ? go(gemv_rows_kernel<DT, B, 32, 4>) : go(gemv_rows_kernel<DT, B, 64, 4>);
        else if (R == 2) rc = lpr == 16 ? go(gemv_rows_kernel<DT, B, 16, 2>) : lpr == 32 ? go(gemv_rows_kernel<DT, B, 32, 2>) : go(gemv_rows_kernel<DT, B, 64, 2>);
        else rc = lpr == 16 ? go(gemv_rows_kernel<DT, B, 16, 1>) : lpr == 32 ? go(gemv_rows_kernel<DT, B, 32, 1>) : go(gemv_rows_kernel<DT, B, 64, 1>);
        if (rc) return rc;
    }
    return AIONHIP_OK;
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
int launch_b(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, int m,
             PreparedAct act, float alpha, float beta) {
    if (m == 1) {
        launch_r<DT, 1>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
        return AIONHIP_OK;
    }
    // q8 with a K too long for one LDS-resident pass: the activation bytes per weight byte are half of q4's, and
    // operands through L1 (gemv_kernel) then beat two sliced launches (measured at 4096 x 14336, 8 rows)
    const int bb = m == 2 ? 2 : (m <= 4 ? 4 : 8);
    if (DT == AIONHIP_Q8_0 && (size_t)bb * 40 * (ws[0]->k >> 5) > ROWS_LDS_CAP) {
        if (bb == 2) launch_r<DT, 2>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
        else if (bb == 4) launch_r<DT, 4>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
        else launch_r<DT, 8>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
        return AIONHIP_OK;
    }
    if (bb == 2) return launch_rows<DT, 2>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
    if (bb == 4) return launch_rows<DT, 4>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
    return launch_rows<DT, 8>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
}

}  // namespace

int launch_gemv_batch(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, int m,
                      PreparedAct act, float alpha, float beta) {
    if (m < 1 || m > 8) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "gemv: m=%d outside 1..8", m);
    if (count < 1 || count > 4) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "gemv: %d weights in one launch (1..4)", count);
    if (gemv_mfma_applies(ws, count, m)) {
        const char *mname = ws[0]->dtype == AIONHIP_Q8_0 ? "gemv_q8_mfma" : "gemv_q4_mfma";
        ProfScope scope(ctx, mname);
        const int rc = launch_gemv_mfma(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
        if (rc == AIONHIP_OK) {
            LAUNCH_CHECK(ctx, mname);
            return AIONHIP_OK;
        }
        if (rc != -1) return rc;
    }
    const char *name = ws[0]->dtype == AIONHIP_Q8_0 ? "gemv_q8" : "gemv_q4";
    ProfScope scope(ctx, name);
    // 5..8 rows against a wide, short weight (a logits head at batch 8): the 16-row MFMA tile of the LDS-staged int8
    // GEMM beats the lane-per-row kernel, whose LDS traffic grows with the rows (262144 x 2048, 8 rows: 77 against
    // 104 us for q4, 110 against 142 us for q8). Long K or few columns leave that kernel's grid too sparse.
    // q8 (twice the weight bytes per row: the lane-per-row kernel leaves its latency floor later) moves there from two
    // rows on once the weight has some 12k columns - 14336 x 4096: 22 -> 20 us at 4 rows, 26.6 -> 20.3 at 8;
    // 16384 x 2048: 15 -> 13.7 at 2-4 rows - but not against the largest weights, which the lane-per-row kernel
    // streams faster at 2-4 rows (65536 x 4096: 58-64 against 70 us).
    const size_t n = ws[0]->n, k = ws[0]->k;
    const bool q8w = ws[0]->dtype == AIONHIP_Q8_0;
    const bool tile16 = (m >= 5 && n >= 16384) || (q8w && m >= 2 && n >= 12288 && n * k <= ((size_t)1 << 27)) ||
                        (q8w && m >= 5 && n >= 8192 && k <= 2048);
    if (count == 1 && tile16 && k >= 256 && k <= 4096) {
        const int rc = launch_gemm_i8_few_rows(ctx, ws[0], (size_t)m, act, cs[0], ldcs[0], alpha, beta);
        if (rc) return rc;
        LAUNCH_CHECK(ctx, name);
        return AIONHIP_OK;
    }
    const int rc = ws[0]->dtype == AIONHIP_Q8_0 ? launch_b<AIONHIP_Q8_0>(ctx, ws, cs, ldcs, count, m, act, alpha, beta)
                                                : launch_b<AIONHIP_Q4_0>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
    if (rc) return rc;
    LAUNCH_CHECK(ctx, name);
    return AIONHIP_OK;
}

int launch_gemv(aionhip_ctx *ctx, const aionhip_weight *w, int m, PreparedAct act, float *c, size_t ldc, float alpha, float beta) {
    return launch_gemv_batch(ctx, &w, &c, &ldc, 1, m, act, alpha, beta);
}
