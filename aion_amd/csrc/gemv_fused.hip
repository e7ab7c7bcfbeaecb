// Single-row decode GEMV with the activation built inside the kernel.
//
// At one activation row every kernel of a decode step is latency-bound, so the int8 activation
// preparation (aion cpu/kernels/matmul_q_i8.zig:187-264) - and, when the caller asks for it, the
// RMSNorm (cpu/exec/layernorm.zig:54-155) or the gelu gate (cpu/exec/elementwise.zig:25-37) that
// produces the activation - runs as a prologue of the GEMV instead of as launches of their own.
// Every workgroup recomputes the (small) activation into LDS with the same arithmetic as the
// stand-alone kernels (same codes, same scales), then streams its weight rows exactly like
// gemv_kernel: one wavefront per R rows, 16-byte chunks per lane, v_dot4_i32_i8, DPP fold. The
// grid is capped at a few workgroups per CU and wavefronts stride over the row groups, so the
// prologue is paid a bounded number of times however many rows the weight has.
// K <= 8192 fits (10 KB of LDS); the callers use it up to K = 4096, beyond which the prologue repeated per
// workgroup costs more than one separate preparation launch.
// Two optional epilogues finish a decode block in the same launch (EPI_ROPE_APPEND, EPI_GATE_QUANT below).
#include "common.h"

#include <type_traits>

namespace {

// NCH = float4 activation chunks per thread (K <= 1024 * NCH). LDS is sized per launch:
// K bytes of codes, K/32 scales, K/32 code sums, 4 reduction slots.
// NT = threads per workgroup (K <= 4 * NT * NCH): 256, or more for the plain preparation - the wavefronts of a workgroup
// share one preparation, and every workgroup reads the whole activation at the same moment.
template <int DT, int R, int PRO, int NCH, int EPI, int NT = 256>
__global__ __launch_bounds__(NT) void gemv_fused_kernel(GemvBatch batch, FusedIn in, int K, float alpha, float beta, FusedEpi epi) {
    static_assert(EPI == EPI_NONE || R == 8, "the epilogues own 4 + 4 rows per wavefront");
    static_assert(NT == 256 || (PRO == PRO_QUANT && EPI == EPI_NONE), "wide workgroups: plain preparation only");
    extern __shared__ __attribute__((aligned(16))) unsigned char s_mem[];
    int *s_aq = (int *)s_mem;
    float *s_scale = (float *)(s_mem + K);
    int *s_sum = (int *)(s_mem + K + (K >> 5) * 4);
    float *s_red = (float *)(s_mem + K + (K >> 5) * 8);
    constexpr int MAX_CH4 = NCH;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave_stride = gridDim.x * (NT / 64);
    // the wavefront index is uniform: read through a scalar, the row-group bookkeeping and the
    // base addresses then stay in scalar registers
    int gwave = blockIdx.x * (EPI == EPI_GATE_QUANT ? 8 : NT / 64) + __builtin_amdgcn_readfirstlane(tid >> 6);
    const int KB = K >> 5;
    constexpr bool Q8 = DT == AIONHIP_Q8_0;
    const int chunks = Q8 ? (K >> 4) : KB;

    // the row group of wavefront index `gw`: segment, first row, row offsets
    struct Group {
        const u32x4 *qs, *qs2;      // qs2 / sc2: rows 4..7 of a gate/up group come from the second weight
        const __half *sc, *sc2;
        float *c;
        int n, row0, seg;
        size_t rowq[R], rows[R];
    };
    auto locate = [&](int gw) {
        Group gr;
        int si = 0;
#pragma unroll
        for (int i = 1; i < 4; ++i)
            if (i < batch.count && gw >= batch.seg[i].first_wave) si = i;
        gr.qs = gr.qs2 = batch.seg[si].qs;
        gr.sc = gr.sc2 = batch.seg[si].sc;
        gr.c = batch.seg[si].c;
        gr.n = batch.seg[si].n;
        gr.seg = si;
        gr.row0 = (gw - batch.seg[si].first_wave) * R;
        if (EPI == EPI_ROPE_APPEND) {
            // task -> (head, first of four pairs): rows head*D + e0 + {0..3} and head*D + D/2 + e0 + {0..3}
            const int per_head = epi.d >> 3, task = gw - batch.seg[si].first_wave;
            gr.row0 = (task / per_head) * epi.d + (task % per_head) * 4;
        }
        if (EPI == EPI_GATE_QUANT) {
            // gw = (task * 2 + sub) * 4 + wavefront: outputs j0 .. j0+3 of the gate (rows 0..3) and the up weight (rows 4..7)
            gr.row0 = (gw >> 2) * 16 + (gw & 3) * 4;
            gr.qs = batch.seg[0].qs;
            gr.sc = batch.seg[0].sc;
            gr.qs2 = batch.seg[1].qs;
            gr.sc2 = batch.seg[1].sc;
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int row = EPI == EPI_ROPE_APPEND ? gr.row0 + (r & 3) + (r >> 2) * (epi.d >> 1)
                          : EPI == EPI_GATE_QUANT ? gr.row0 + (r & 3)
                          : min(gr.row0 + r, gr.n - 1);
            gr.rowq[r] = (size_t)row * chunks;
            gr.rows[r] = (size_t)row * KB;
        }
        return gr;
    };
    bool active = gwave < batch.total_waves;
    Group cur = locate(active ? gwave : 0);
    // ---- prologue: activation -> int8 codes, per-block scale and code sum in LDS
    const int n4 = K >> 2;
    f32x4 v[MAX_CH4], aux[PRO == PRO_QUANT ? 1 : MAX_CH4], aux2[PRO == PRO_RMSNORM ? MAX_CH4 : 1];
    // every global operand of the prologue is requested up front: one memory latency, not three
#pragma unroll
    for (int i = 0; i < MAX_CH4; ++i) {
        const int c4 = tid + NT * i;
        const bool live = c4 < n4;
        v[i] = live ? *(const f32x4 *)(in.x + (size_t)c4 * 4) : f32x4{0.f, 0.f, 0.f, 0.f};
        if (PRO == PRO_RMSNORM) {
            aux[i] = live ? *(const f32x4 *)(in.gamma + (size_t)c4 * 4) : f32x4{0.f, 0.f, 0.f, 0.f};
            aux2[i] = (live && in.beta) ? *(const f32x4 *)(in.beta + (size_t)c4 * 4) : f32x4{0.f, 0.f, 0.f, 0.f};
        } else if (PRO == PRO_GATE) {
            aux[i] = live ? *(const f32x4 *)(in.y + (size_t)c4 * 4) : f32x4{0.f, 0.f, 0.f, 0.f};
        }
    }
    // first weight chunk of every row: requested right behind the activation operands (loads return
    // in order, so the prologue waits for the activation only while these stay in flight)
    // (unconditional loads at clamped addresses: predicated loads would be waited for one by one)
    u32x4 w0[R];
    __half hs0[R];
    const bool lane_has0 = lane < chunks;
    const int l0 = min(lane, chunks - 1);
#pragma unroll
    for (int r = 0; r < R; ++r) {
        w0[r] = __builtin_nontemporal_load((EPI == EPI_GATE_QUANT && r >= 4 ? cur.qs2 : cur.qs) + cur.rowq[r] + l0);
        hs0[r] = (EPI == EPI_GATE_QUANT && r >= 4 ? cur.sc2 : cur.sc)[cur.rows[r] + (Q8 ? (l0 >> 1) : l0)];
    }

    float ss = 0.f;
    if (PRO == PRO_RMSNORM) {
#pragma unroll
        for (int i = 0; i < MAX_CH4; ++i) ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
    }
    float inv_rms = 1.f;
    if (PRO == PRO_RMSNORM) {
        ss = block_sum_256(ss, s_red);
        inv_rms = 1.f / sqrtf(ss * (1.f / (float)K) + in.eps);
    }
#pragma unroll
    for (int i = 0; i < MAX_CH4; ++i) {
        const int c4 = tid + NT * i;
        const bool live = c4 < n4;
        f32x4 a = v[i];
        if (live) {
            if (PRO == PRO_RMSNORM) {
                const f32x4 gm = aux[i], bt = aux2[i];
                a.x = (a.x * inv_rms) * gm.x + bt.x;
                a.y = (a.y * inv_rms) * gm.y + bt.y;
                a.z = (a.z * inv_rms) * gm.z + bt.z;
                a.w = (a.w * inv_rms) * gm.w + bt.w;
            } else if (PRO == PRO_GATE) {
                const f32x4 up = aux[i];
                a.x = aion_gate_gelu(a.x, up.x);
                a.y = aion_gate_gelu(a.y, up.y);
                a.z = aion_gate_gelu(a.z, up.z);
                a.w = aion_gate_gelu(a.w, up.w);
            }
        }
        // 8 consecutive lanes share one 32-element block (c4 >> 3)
        int word, s;
        float scale;
        prepare_act_block8(a.x, a.y, a.z, a.w, word, scale, s);
        if (live) {
            s_aq[c4] = word;
            if ((c4 & 7) == 0) {
                s_scale[c4 >> 3] = scale;
                s_sum[c4 >> 3] = s;
            }
        }
    }
    __syncthreads();

    // ---- stream the row groups
    const u32x4 *aq = (const u32x4 *)s_aq;
    while (active) {
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; ++r) acc[r] = 0.f;

        auto consume = [&](int ch, const u32x4 (&w)[R], const float (&ws)[R]) {
            const int blk = Q8 ? (ch >> 1) : ch;
            const float as = s_scale[blk];
            if (Q8) {
                const u32x4 a = aq[ch];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    int d = dot4_i8((int)a.x, (int)w[r].x, 0);
                    d = dot4_i8((int)a.y, (int)w[r].y, d);
                    d = dot4_i8((int)a.z, (int)w[r].z, d);
                    d = dot4_i8((int)a.w, (int)w[r].w, d);
                    acc[r] += (float)d * (as * ws[r]);
                }
            } else {
                const u32x4 a0 = aq[2 * ch], a1 = aq[2 * ch + 1];
                const int bias = 8 * s_sum[blk];
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
                    acc[r] += (float)d * (as * ws[r]);
                }
            }
        };

        if (lane_has0) {
            float ws0[R];
#pragma unroll
            for (int r = 0; r < R; ++r) ws0[r] = __half2float(hs0[r]);
            consume(lane, w0, ws0);
        }
        // the remaining chunks, U at a time with all U*R loads in flight before the first is consumed
        constexpr int U = R == 1 ? 4 : (R == 2 ? 2 : 1);
#pragma unroll 1
        for (int ch0 = lane + 64; ch0 < chunks; ch0 += 64 * U) {
            u32x4 w[U][R];
            __half hs[U][R];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int ch = min(ch0 + 64 * u, chunks - 1);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    w[u][r] = __builtin_nontemporal_load((EPI == EPI_GATE_QUANT && r >= 4 ? cur.qs2 : cur.qs) + cur.rowq[r] + ch);
                    hs[u][r] = (EPI == EPI_GATE_QUANT && r >= 4 ? cur.sc2 : cur.sc)[cur.rows[r] + (Q8 ? (ch >> 1) : ch)];
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (ch0 + 64 * u < chunks) {
                    float ws[R];
#pragma unroll
                    for (int r = 0; r < R; ++r) ws[r] = __half2float(hs[u][r]);
                    consume(ch0 + 64 * u, w[u], ws);
                }
            }
        }

#pragma unroll
        for (int r = 0; r < R; ++r) acc[r] = wave_sum(acc[r]);
        if (EPI == EPI_ROPE_APPEND) {
            // every lane holds all eight sums; lane p < 4 finishes pair p (aion cpu/kernels/rope.zig:20-98,
            // cpu/exec/cast.zig, cpu/exec/sequence_append.zig:12-104 - the arithmetic of rope_append_kernel)
            if (lane < 4) {
                const float xl = alpha * (lane == 0 ? acc[0] : lane == 1 ? acc[1] : lane == 2 ? acc[2] : acc[3 % R]);
                const float xh = alpha * (lane == 0 ? acc[4 % R] : lane == 1 ? acc[5 % R] : lane == 2 ? acc[6 % R] : acc[7 % R]);
                const int half = epi.d >> 1;
                const int head = cur.row0 / epi.d, i = cur.row0 % epi.d + lane;      // i < D/2
                const bool rot = cur.seg < 2 && i < epi.rope_pairs;
                float sn = 0.f, cs = 1.f;
                if (rot) sincosf((float)epi.positions[0] * epi.freq[i], &sn, &cs);
                float yl = xl, yh = xh;
                if (rot) rope_rotate(xl, xh, sn, cs, yl, yh);
                if (cur.seg == 0) {
                    cur.c[head * epi.d + i] = yl;
                    cur.c[head * epi.d + half + i] = yh;
                } else {
                    long t = (long)epi.write_index[0];
                    if (epi.rolling && t >= 0) t %= (long)epi.t_cap;                  // storage/cache.zig:202-207
                    if (t >= 0 && t < (long)epi.t_cap) {                               // never write outside the cache
                        __half *dst = (cur.seg == 1 ? epi.k_cache : epi.v_cache) + ((size_t)t * epi.h_kv + head) * epi.d;
                        dst[i] = __float2half_rn(yl);
                        dst[half + i] = __float2half_rn(yh);
                    }
                }
            }
        } else if (EPI == EPI_GATE_QUANT) {
            // lanes 0..3: h_j; after the second 16 outputs the workgroup's 32 values are one quant block
            float *s_h = s_red + 4;
            if (lane < 4) {
                const float gv = alpha * (lane == 0 ? acc[0] : lane == 1 ? acc[1] : lane == 2 ? acc[2] : acc[3 % R]);
                const float uv = alpha * (lane == 0 ? acc[4 % R] : lane == 1 ? acc[5 % R] : lane == 2 ? acc[6 % R] : acc[7 % R]);
                s_h[(cur.row0 & 31) + lane] = aion_gate_gelu(gv, uv);       // row0 & 31 = sub * 16 + wavefront * 4
            }
            if ((gwave >> 2) & 1) {
                __syncthreads();
                if (tid < 8) {
                    // the shared block preparation (aion cpu/kernels/matmul_q_i8.zig:187-203), 8 lanes x 4 values
                    const float v0 = s_h[tid * 4], v1 = s_h[tid * 4 + 1], v2 = s_h[tid * 4 + 2], v3 = s_h[tid * 4 + 3];
                    int word, sq;
                    float scale;
                    prepare_act_block8(v0, v1, v2, v3, word, scale, sq);
                    const int blk = gwave >> 3;                     // task = quant block of the down projection's activation
                    epi.act_q[blk * 8 + tid] = word;
                    if (tid == 0) {
                        epi.act_scale[blk] = scale;
                        epi.act_sum[blk] = sq;
                    }
                }
                __syncthreads();                                    // s_h is reused by the next task
            }
        } else if (lane == 0) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (cur.row0 + r >= cur.n) break;
                const float val = alpha * acc[r];
                cur.c[cur.row0 + r] = beta == 0.f ? val : val + beta * cur.c[cur.row0 + r];
            }
        }
        if (EPI == EPI_GATE_QUANT) gwave = ((gwave >> 2) & 1) ? gwave - 4 + 8 * (int)gridDim.x : gwave + 4;
        else gwave += wave_stride;
        active = gwave < batch.total_waves;
        if (active) {
            cur = locate(gwave);
#pragma unroll
            for (int r = 0; r < R; ++r) {
                w0[r] = __builtin_nontemporal_load((EPI == EPI_GATE_QUANT && r >= 4 ? cur.qs2 : cur.qs) + cur.rowq[r] + l0);
                hs0[r] = (EPI == EPI_GATE_QUANT && r >= 4 ? cur.sc2 : cur.sc)[cur.rows[r] + (Q8 ? (l0 >> 1) : l0)];
            }
        }
    }
}

template <int DT, int PRO, int NCH>
void launch_r(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, FusedIn in,
              float alpha, float beta) {
    const int K = (int)ws[0]->k;
    long n_total = 0;
    for (int i = 0; i < count; ++i) n_total += (long)ws[i]->n;
    const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
    int R = 4;
    if (n_total < (long)cus * 8 * 4) R = 2;
    if (n_total < (long)cus * 8 * 2) R = 1;
    GemvBatch batch{};
    batch.count = count;
    int waves = 0;
    for (int i = 0; i < count; ++i) {
        batch.seg[i] = GemvSeg{(const u32x4 *)ws[i]->qs, ws[i]->sc, cs[i], ldcs[i], (int)ws[i]->n, waves};
        waves += ((int)ws[i]->n + R - 1) / R;
    }
    batch.total_waves = waves;
    const size_t lds = (size_t)K + (size_t)(K >> 5) * 8 + 16;
    if constexpr (PRO == PRO_QUANT) {
        // The plain preparation runs in wide workgroups (1024 threads: sixteen wavefronts share one preparation, and fewer
        // workgroups hit the activation's few L2 lines at the same moment; q4, one row: 4096x4096 5.3 -> 4.6 us,
        // 14336x4096 8.7 -> 7.8 us) on a grid capped at 32 wavefronts per CU, whose wavefronts stride over the row groups.
        // A weight with many more row groups than that (a logits head) gets 512-thread workgroups and up to eight rounds of
        // them before the striding starts: the hardware then deals workgroups out as CUs free up, which evens out the tail
        // (262144x2048: 45.8 -> 44 us back to back, 46 -> 45 us between other kernels).
        const bool many = waves > cus * 64;
        const int nt = many ? 512 : 1024, rounds = many ? 8 : 1;
        auto go = [&](auto nt_tag) {
            constexpr int WNT = decltype(nt_tag)::value, WNCH = (NCH * 256 + WNT - 1) / WNT;
            const int wg = (waves + WNT / 64 - 1) / (WNT / 64), cap = cus * 32 / (WNT / 64) * rounds;
            const dim3 wgrid((unsigned)(wg < cap ? wg : cap)), wblock(WNT);
            if (R == 4) launch_k(ctx, gemv_fused_kernel<DT, 4, PRO_QUANT, WNCH, EPI_NONE, WNT>, wgrid, wblock, lds, batch, in, K, alpha, beta, FusedEpi{});
            else if (R == 2) launch_k(ctx, gemv_fused_kernel<DT, 2, PRO_QUANT, WNCH, EPI_NONE, WNT>, wgrid, wblock, lds, batch, in, K, alpha, beta, FusedEpi{});
            else launch_k(ctx, gemv_fused_kernel<DT, 1, PRO_QUANT, WNCH, EPI_NONE, WNT>, wgrid, wblock, lds, batch, in, K, alpha, beta, FusedEpi{});
        };
        if (nt == 512) go(std::integral_constant<int, 512>{});
        else go(std::integral_constant<int, 1024>{});
    } else {
        // at most 8 workgroups per CU: beyond that the wavefronts stride over the row groups (more rounds of workgroups,
        // as for the plain preparation above, cost more here than they even out: every workgroup redoes the norm's
        // reduction; 262144x2048 behind an RMSNorm: 50.8 us on this grid, 56.7 us on eight rounds)
        const int wgs = (waves + 3) / 4;
        const dim3 grid((unsigned)(wgs < cus * 8 ? wgs : cus * 8)), block(256);
        if (R == 4) launch_k(ctx, gemv_fused_kernel<DT, 4, PRO, NCH, EPI_NONE>, grid, block, lds, batch, in, K, alpha, beta, FusedEpi{});
        else if (R == 2) launch_k(ctx, gemv_fused_kernel<DT, 2, PRO, NCH, EPI_NONE>, grid, block, lds, batch, in, K, alpha, beta, FusedEpi{});
        else launch_k(ctx, gemv_fused_kernel<DT, 1, PRO, NCH, EPI_NONE>, grid, block, lds, batch, in, K, alpha, beta, FusedEpi{});
    }
}

template <int DT, int PRO>
void launch_n(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, FusedIn in,
              float alpha, float beta) {
    const size_t k = ws[0]->k;
    if (k <= 2048) launch_r<DT, PRO, 2>(ctx, ws, cs, ldcs, count, in, alpha, beta);
    else if (k <= 4096) launch_r<DT, PRO, 4>(ctx, ws, cs, ldcs, count, in, alpha, beta);
    else launch_r<DT, PRO, 8>(ctx, ws, cs, ldcs, count, in, alpha, beta);
}

template <int DT>
void launch_p(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, int pro, FusedIn in,
              float alpha, float beta) {
    if (pro == PRO_RMSNORM) launch_n<DT, PRO_RMSNORM>(ctx, ws, cs, ldcs, count, in, alpha, beta);
    else if (pro == PRO_GATE) launch_n<DT, PRO_GATE>(ctx, ws, cs, ldcs, count, in, alpha, beta);
    else launch_n<DT, PRO_QUANT>(ctx, ws, cs, ldcs, count, in, alpha, beta);
}

template <int DT, int NCH>
void launch_rope(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *q_out, FusedIn in, FusedEpi epi) {
    const int K = (int)ws[0]->k;
    GemvBatch batch{};
    batch.count = 3;
    int waves = 0;
    for (int i = 0; i < 3; ++i) {
        batch.seg[i] = GemvSeg{(const u32x4 *)ws[i]->qs, ws[i]->sc, i == 0 ? q_out : nullptr, ws[i]->n, (int)ws[i]->n, waves};
        waves += (int)ws[i]->n / 8;
    }
    batch.total_waves = waves;
    const dim3 grid((unsigned)((waves + 3) / 4)), block(256);
    const size_t lds = (size_t)K + (size_t)(K >> 5) * 8 + 16;
    launch_k(ctx, gemv_fused_kernel<DT, 8, PRO_RMSNORM, NCH, EPI_ROPE_APPEND>, grid, block, lds, batch, in, K, 1.f, 0.f, epi);
}

template <int DT, int NCH>
void launch_geglu(aionhip_ctx *ctx, const aionhip_weight *gate, const aionhip_weight *up, FusedIn in, PreparedAct out) {
    const int K = (int)gate->k, tasks = (int)gate->n / 32;
    GemvBatch batch{};
    batch.count = 2;
    batch.seg[0] = GemvSeg{(const u32x4 *)gate->qs, gate->sc, nullptr, gate->n, (int)gate->n, 0};
    batch.seg[1] = GemvSeg{(const u32x4 *)up->qs, up->sc, nullptr, up->n, (int)up->n, 0};
    batch.total_waves = tasks * 8;
    const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
    const dim3 grid((unsigned)(tasks < cus * 8 ? tasks : cus * 8)), block(256);
    const size_t lds = (size_t)K + (size_t)(K >> 5) * 8 + 16 + 32 * sizeof(float);
    FusedEpi epi{};
    epi.act_q = (int *)out.q;
    epi.act_scale = out.scale;
    epi.act_sum = out.sum;
    launch_k(ctx, gemv_fused_kernel<DT, 8, PRO_RMSNORM, NCH, EPI_GATE_QUANT>, grid, block, lds, batch, in, K, 1.f, 0.f, epi);
}

}  // namespace

int launch_gemv_fused_geglu(aionhip_ctx *ctx, const aionhip_weight *gate, const aionhip_weight *up, FusedIn in, PreparedAct out) {
    const bool q8 = gate->dtype == AIONHIP_Q8_0;
    const char *name = q8 ? "gemv_q8_rmsnorm_geglu" : "gemv_q4_rmsnorm_geglu";
    ProfScope scope(ctx, name);
    const size_t k = gate->k;
    if (q8) {
        if (k <= 2048) launch_geglu<AIONHIP_Q8_0, 2>(ctx, gate, up, in, out);
        else if (k <= 4096) launch_geglu<AIONHIP_Q8_0, 4>(ctx, gate, up, in, out);
        else launch_geglu<AIONHIP_Q8_0, 8>(ctx, gate, up, in, out);
    } else {
        if (k <= 2048) launch_geglu<AIONHIP_Q4_0, 2>(ctx, gate, up, in, out);
        else if (k <= 4096) launch_geglu<AIONHIP_Q4_0, 4>(ctx, gate, up, in, out);
        else launch_geglu<AIONHIP_Q4_0, 8>(ctx, gate, up, in, out);
    }
    LAUNCH_CHECK(ctx, name);
    return AIONHIP_OK;
}

int launch_gemv_fused_rope(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *q_out, FusedIn in, FusedEpi epi) {
    const bool q8 = ws[0]->dtype == AIONHIP_Q8_0;
    const char *name = q8 ? "gemv_q8_rmsnorm_rope" : "gemv_q4_rmsnorm_rope";
    ProfScope scope(ctx, name);
    const size_t k = ws[0]->k;
    if (q8) {
        if (k <= 2048) launch_rope<AIONHIP_Q8_0, 2>(ctx, ws, q_out, in, epi);
        else if (k <= 4096) launch_rope<AIONHIP_Q8_0, 4>(ctx, ws, q_out, in, epi);
        else launch_rope<AIONHIP_Q8_0, 8>(ctx, ws, q_out, in, epi);
    } else {
        if (k <= 2048) launch_rope<AIONHIP_Q4_0, 2>(ctx, ws, q_out, in, epi);
        else if (k <= 4096) launch_rope<AIONHIP_Q4_0, 4>(ctx, ws, q_out, in, epi);
        else launch_rope<AIONHIP_Q4_0, 8>(ctx, ws, q_out, in, epi);
    }
    LAUNCH_CHECK(ctx, name);
    return AIONHIP_OK;
}

int launch_gemv_fused(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, int prologue,
                      FusedIn in, float alpha, float beta) {
    if (count < 1 || count > 4) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "gemv: %d weights in one launch (1..4)", count);
    if (ws[0]->k > FUSED_MAX_K) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "fused gemv: k=%zu exceeds %zu", ws[0]->k, FUSED_MAX_K);
    if (((uintptr_t)in.x & 15) || ((uintptr_t)in.y & 15) || ((uintptr_t)in.gamma & 15) || ((uintptr_t)in.beta & 15))
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "fused gemv: activation operands must be 16-byte aligned");
    static const char *names[2][3] = {{"gemv_q4_fused", "gemv_q4_rmsnorm", "gemv_q4_gate"}, {"gemv_q8_fused", "gemv_q8_rmsnorm", "gemv_q8_gate"}};
    const bool q8 = ws[0]->dtype == AIONHIP_Q8_0;
    const char *name = names[q8 ? 1 : 0][prologue];
    ProfScope scope(ctx, name);
    if (q8) launch_p<AIONHIP_Q8_0>(ctx, ws, cs, ldcs, count, prologue, in, alpha, beta);
    else launch_p<AIONHIP_Q4_0>(ctx, ws, cs, ldcs, count, prologue, in, alpha, beta);
    LAUNCH_CHECK(ctx, name);
    return AIONHIP_OK;
}
