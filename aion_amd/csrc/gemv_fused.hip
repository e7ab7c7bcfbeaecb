// Single-row decode GEMV with the activation built inside the kernel.
//
// At one activation row every kernel of a decode step is latency-bound, so the int8 activation
// preparation (aion cpu/kernels/matmul_q_i8.zig:187-264) - and, when the caller asks for it, the
// RMSNorm (cpu/exec/layernorm.zig:54-155) or the gelu gate (cpu/exec/elementwise.zig:25-37) that
// produces the activation - runs as a prologue of the GEMV instead of as launches of their own.
// Every workgroup recomputes the (small) activation into LDS with the same arithmetic as the
// stand-alone kernels (same codes, same scales), then streams its weight rows exactly like
// gemv_kernel: one wavefront per R rows, 16-byte chunks per lane, v_dot4_i32_i8, DPP fold.
// K <= 8192 (10 KB of LDS); larger K keeps the separate preparation launch.
#include "common.h"

namespace {

constexpr int MAX_CH4 = (int)(FUSED_MAX_K / 4 / 256);   // float4 chunks per thread

template <int DT, int R, int PRO>
__global__ __launch_bounds__(256) void gemv_fused_kernel(GemvBatch batch, FusedIn in, int K, float alpha, float beta) {
    __shared__ __attribute__((aligned(16))) int s_aq[FUSED_MAX_K / 4];
    __shared__ float s_scale[FUSED_MAX_K / QK];
    __shared__ int s_sum[FUSED_MAX_K / QK];
    __shared__ float s_red[4];

    const int tid = threadIdx.x, lane = tid & 63;
    const int gwave = blockIdx.x * 4 + (tid >> 6);
    const bool active = gwave < batch.total_waves;
    int si = 0;
#pragma unroll
    for (int i = 1; i < 4; ++i)
        if (i < batch.count && gwave >= batch.seg[i].first_wave) si = i;
    const u32x4 *__restrict__ qs = batch.seg[si].qs;
    const __half *__restrict__ sc = batch.seg[si].sc;
    const int N = batch.seg[si].n;
    const int row0 = active ? (gwave - batch.seg[si].first_wave) * R : 0;
    const int KB = K >> 5;
    constexpr bool Q8 = DT == AIONHIP_Q8_0;
    const int chunks = Q8 ? (K >> 4) : KB;

    size_t rowq[R], rows[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int row = min(row0 + r, N - 1);
        rowq[r] = (size_t)row * chunks;
        rows[r] = (size_t)row * KB;
    }
    // first weight chunk of every row: issued before the prologue so that its latency overlaps it
    u32x4 w0[R];
    float ws0[R];
    const bool have0 = active && lane < chunks;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        w0[r] = have0 ? __builtin_nontemporal_load(qs + rowq[r] + lane) : u32x4{0u, 0u, 0u, 0u};
        ws0[r] = have0 ? __half2float(sc[rows[r] + (Q8 ? (lane >> 1) : lane)]) : 0.f;
    }

    // ---- prologue: activation -> int8 codes, per-block scale and code sum in LDS
    const int n4 = K >> 2;
    f32x4 v[MAX_CH4];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < MAX_CH4; ++i) {
        const int c4 = tid + 256 * i;
        v[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (c4 < n4) {
            v[i] = *(const f32x4 *)(in.x + (size_t)c4 * 4);
            if (PRO == PRO_RMSNORM) ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
        }
    }
    float inv_rms = 1.f;
    if (PRO == PRO_RMSNORM) {
        ss = block_sum_256(ss, s_red);
        inv_rms = 1.f / sqrtf(ss * (1.f / (float)K) + in.eps);
    }
#pragma unroll
    for (int i = 0; i < MAX_CH4; ++i) {
        const int c4 = tid + 256 * i;
        const bool live = c4 < n4;
        f32x4 a = v[i];
        if (live) {
            if (PRO == PRO_RMSNORM) {
                const f32x4 gm = *(const f32x4 *)(in.gamma + (size_t)c4 * 4);
                f32x4 bt = f32x4{0.f, 0.f, 0.f, 0.f};
                if (in.beta) bt = *(const f32x4 *)(in.beta + (size_t)c4 * 4);
                a.x = (a.x * inv_rms) * gm.x + bt.x;
                a.y = (a.y * inv_rms) * gm.y + bt.y;
                a.z = (a.z * inv_rms) * gm.z + bt.z;
                a.w = (a.w * inv_rms) * gm.w + bt.w;
            } else if (PRO == PRO_GATE) {
                const f32x4 up = *(const f32x4 *)(in.y + (size_t)c4 * 4);
                a.x = aion_gate_gelu(a.x, up.x);
                a.y = aion_gate_gelu(a.y, up.y);
                a.z = aion_gate_gelu(a.z, up.z);
                a.w = aion_gate_gelu(a.w, up.w);
            }
        }
        // 8 consecutive lanes share one 32-element block (c4 >> 3)
        float amax = fmaxf(fmaxf(fabsf(a.x), fabsf(a.y)), fmaxf(fabsf(a.z), fabsf(a.w)));
        amax = fmaxf(amax, dpp_f<DPP_QUAD_XOR1>(amax));
        amax = fmaxf(amax, dpp_f<DPP_QUAD_XOR2>(amax));
        amax = fmaxf(amax, dpp_f<DPP_ROW_HALF_MIRROR>(amax));
        int word = 0, s = 0;
        float scale = 0.f;
        if (amax != 0.f) {
            scale = amax / 127.f;
            const float inv = 127.f / amax;
            const int q0 = (int)fminf(127.f, fmaxf(-127.f, roundf(a.x * inv)));
            const int q1 = (int)fminf(127.f, fmaxf(-127.f, roundf(a.y * inv)));
            const int q2 = (int)fminf(127.f, fmaxf(-127.f, roundf(a.z * inv)));
            const int q3 = (int)fminf(127.f, fmaxf(-127.f, roundf(a.w * inv)));
            word = (q0 & 0xFF) | ((q1 & 0xFF) << 8) | ((q2 & 0xFF) << 16) | ((q3 & 0xFF) << 24);
            s = q0 + q1 + q2 + q3;
        }
        s += dpp_i<DPP_QUAD_XOR1>(s);
        s += dpp_i<DPP_QUAD_XOR2>(s);
        s += dpp_i<DPP_ROW_HALF_MIRROR>(s);
        if (live) {
            s_aq[c4] = word;
            if ((c4 & 7) == 0) {
                s_scale[c4 >> 3] = scale;
                s_sum[c4 >> 3] = s;
            }
        }
    }
    __syncthreads();
    if (!active) return;

    // ---- stream the rows
    const u32x4 *aq = (const u32x4 *)s_aq;
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

    if (have0) consume(lane, w0, ws0);
#pragma unroll 2
    for (int ch = lane + 64; ch < chunks; ch += 64) {
        u32x4 w[R];
        float ws[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            w[r] = __builtin_nontemporal_load(qs + rowq[r] + ch);
            ws[r] = __half2float(sc[rows[r] + (Q8 ? (ch >> 1) : ch)]);
        }
        consume(ch, w, ws);
    }

#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = wave_sum(acc[r]);
    if (lane == 0) {
        float *c = batch.seg[si].c;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (row0 + r >= N) break;
            const float val = alpha * acc[r];
            c[row0 + r] = beta == 0.f ? val : val + beta * c[row0 + r];
        }
    }
}

template <int DT, int PRO>
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
    const dim3 grid((unsigned)((waves + 3) / 4)), block(256);
    if (R == 4) gemv_fused_kernel<DT, 4, PRO><<<grid, block, 0, ctx->stream>>>(batch, in, K, alpha, beta);
    else if (R == 2) gemv_fused_kernel<DT, 2, PRO><<<grid, block, 0, ctx->stream>>>(batch, in, K, alpha, beta);
    else gemv_fused_kernel<DT, 1, PRO><<<grid, block, 0, ctx->stream>>>(batch, in, K, alpha, beta);
}

template <int DT>
void launch_p(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, int pro, FusedIn in,
              float alpha, float beta) {
    if (pro == PRO_RMSNORM) launch_r<DT, PRO_RMSNORM>(ctx, ws, cs, ldcs, count, in, alpha, beta);
    else if (pro == PRO_GATE) launch_r<DT, PRO_GATE>(ctx, ws, cs, ldcs, count, in, alpha, beta);
    else launch_r<DT, PRO_QUANT>(ctx, ws, cs, ldcs, count, in, alpha, beta);
}

}  // namespace

int launch_gemv_fused(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, int prologue,
                      FusedIn in, float alpha, float beta) {
    if (count < 1 || count > 4) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "gemv: %d weights in one launch (1..4)", count);
    if (ws[0]->k > FUSED_MAX_K) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "fused gemv: k=%zu exceeds %zu", ws[0]->k, FUSED_MAX_K);
    if (((uintptr_t)in.x & 15) || ((uintptr_t)in.y & 15) || ((uintptr_t)in.gamma & 15) || ((uintptr_t)in.beta & 15))
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "fused gemv: activation operands must be 16-byte aligned");
    static const char *names[2][3] = {{"gemv_q4_fused", "gemv_q4_rmsnorm", "gemv_q4_gate"}, {"gemv_q8_fused", "gemv_q8_rmsnorm", "gemv_q8_gate"}};
    const bool q8 = ws[0]->dtype == AIONHIP_Q8_0;
    const char *name = names[q8 ? 1 : 0][prologue];
    prof_begin(ctx, name);
    if (q8) launch_p<AIONHIP_Q8_0>(ctx, ws, cs, ldcs, count, prologue, in, alpha, beta);
    else launch_p<AIONHIP_Q4_0>(ctx, ws, cs, ldcs, count, prologue, in, alpha, beta);
    prof_end(ctx);
    LAUNCH_CHECK(ctx, name);
    return AIONHIP_OK;
}
