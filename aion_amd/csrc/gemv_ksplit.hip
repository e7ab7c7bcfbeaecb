// Single-row decode GEMV for a long reduction axis (K > 4096): the K axis is cut into slices and a workgroup owns
// (a group of weight rows) x (one K slice).
//
// Why: with the whole K in one workgroup every workgroup would have to prepare the whole activation (tens of KB read by
// hundreds of workgroups at the same moment: the loads pile up on the same L2 channels), which is why long rows used to
// run as a separate preparation launch followed by the GEMV - two dependent launches, and with few rows (N = 4096) too
// few wavefronts to keep the memory system busy. Here a workgroup prepares only its own slice of the activation
// (aion cpu/kernels/matmul_q_i8.zig:187-264, the shared block preparation) into LDS, so the activation is read S times
// less per workgroup, there are S times more wavefronts, and there is one launch.
//
// The S partial sums of a row (S a power of two) are combined without float atomics and without a second launch, along a
// fixed binary tree: slices 2j and 2j+1 meet in a 64-bit word {flag, partial}. A wavefront swaps its partial in with one
// device-scope atomic exchange; if the word was empty it is done (its partial is parked there), otherwise it got the
// sibling's partial back, adds the two in slice order (even + odd, whoever came second), empties the word again and
// carries the sum to the next level. The sum is ((p0+p1)+(p2+p3))+... whatever the arrival order, so the result does not
// depend on timing; the worst-case chain is log2(S) memory round trips, and every word is empty again when the launch
// ends. aion's own K-major matvec walks long rows in chunks too (cpu/kernels/matvec_q.zig:87-97: chunk 0 stores
// alpha * dot + beta * C, later chunks add); only the order of the f32 additions differs.
#include "common.h"

namespace {

constexpr int KSPLIT_MAX_S = 8;

// CPL: 16-byte weight chunks per lane per row in one slice (the slice has at most 64 * CPL chunks); all of them are requested
// before the activation is prepared, so a wavefront pays one memory round trip for its weights, overlapped with the
// round trip of the activation slice. NCH: float4 activation chunks per thread (the slice has at most 4 * NT * NCH floats).
template <int DT, int R, int NT, int NCH, int CPL>
__global__ __launch_bounds__(NT) void gemv_ksplit_kernel(const u32x4 *__restrict__ qs, const __half *__restrict__ sc, float *__restrict__ c,
                                                         const float *__restrict__ x, unsigned long long *meet, int N, int K, int kbs, int S, int groups, int interleave,
                                                         float alpha, float beta) {
    extern __shared__ __attribute__((aligned(16))) unsigned char s_mem[];
    constexpr bool Q8 = DT == AIONHIP_Q8_0;
    constexpr int WPB = NT / 64;                            // wavefronts per workgroup
    int *s_aq = (int *)s_mem;                               // kbs * 32 bytes of codes
    float *s_scale = (float *)(s_mem + kbs * 32);
    int *s_sum = (int *)(s_mem + kbs * 36);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // workgroup -> (row group, slice). Slice-major (all row groups of slice 0 first) is the faster order in general. Where
    // the row pitch is a multiple of 8 KiB, a slice is the same 2 KiB column range of every row, and a dispatch order that
    // works through one slice at a time keeps hitting the same quarter of the memory channels; there the slices alternate from
    // one workgroup to the next, rotated every 8 / S row groups so that one XCD (every eighth workgroup) sees all of them.
    const int b_lin = blockIdx.x;
    int g, s;
    if (interleave) {
        g = b_lin / S;
        s = (b_lin % S + g / (S >= 8 ? 1 : 8 / S)) % S;
    } else {
        g = b_lin % groups;
        s = b_lin / groups;
    }
    const int KB = K >> 5, kb0 = s * kbs, kbn = min(kbs, KB - kb0);
    const int gw = g * WPB + wave;                          // this wavefront's row group
    const int row0 = gw * R;
    const int chunks_row = Q8 ? (K >> 4) : KB;              // 16-byte weight chunks per full row
    const int ch0 = Q8 ? 2 * kb0 : kb0, nch = Q8 ? 2 * kbn : kbn;

    // this slice of the activation first, all weight chunks of the wavefront's rows right behind it (unconditional loads at
    // clamped addresses: a predicated load would be waited for on the spot)
    const int n4 = kbn * 8;
    f32x4 v[NCH];
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int c4 = tid + NT * i;
        v[i] = *(const f32x4 *)(x + (size_t)kb0 * 32 + (size_t)min(c4, n4 - 1) * 4);
    }
    u32x4 w[CPL][R];
    __half hs[CPL][R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int row = min(row0 + r, N - 1);
        const u32x4 *__restrict__ wq = qs + (size_t)row * chunks_row + ch0;
        const __half *__restrict__ wsc = sc + (size_t)row * KB + kb0;
#pragma unroll
        for (int u = 0; u < CPL; ++u) {
            const int ch = min(lane + 64 * u, nch - 1);
            w[u][r] = __builtin_nontemporal_load(wq + ch);
            hs[u][r] = wsc[Q8 ? (ch >> 1) : ch];
        }
    }
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int c4 = tid + NT * i;
        int word, sm;
        float scale;
        prepare_act_block8(v[i].x, v[i].y, v[i].z, v[i].w, word, scale, sm);
        if (c4 < n4) {
            s_aq[c4] = word;
            if ((c4 & 7) == 0) {
                s_scale[c4 >> 3] = scale;
                s_sum[c4 >> 3] = sm;
            }
        }
    }
    __syncthreads();

    const u32x4 *aq = (const u32x4 *)s_aq;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;
#pragma unroll
    for (int u = 0; u < CPL; ++u) {
        const int ch = lane + 64 * u;
        if (ch < nch) {
            const int blk = Q8 ? (ch >> 1) : ch;
            const float as = s_scale[blk];
            if (Q8) {
                const u32x4 a = aq[ch];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    int d = dot4_i8((int)a.x, (int)w[u][r].x, 0);
                    d = dot4_i8((int)a.y, (int)w[u][r].y, d);
                    d = dot4_i8((int)a.z, (int)w[u][r].z, d);
                    d = dot4_i8((int)a.w, (int)w[u][r].w, d);
                    acc[r] += (float)d * (as * __half2float(hs[u][r]));
                }
            } else {
                const u32x4 a0 = aq[2 * ch], a1 = aq[2 * ch + 1];
                const int bias = 8 * s_sum[blk];             // codes are nibble - 8
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    constexpr unsigned M = 0x0F0F0F0Fu;
                    int d = dot4_i8((int)a0.x, (int)(w[u][r].x & M), -bias);
                    d = dot4_i8((int)a0.y, (int)((w[u][r].x >> 4) & M), d);
                    d = dot4_i8((int)a0.z, (int)(w[u][r].y & M), d);
                    d = dot4_i8((int)a0.w, (int)((w[u][r].y >> 4) & M), d);
                    d = dot4_i8((int)a1.x, (int)(w[u][r].z & M), d);
                    d = dot4_i8((int)a1.y, (int)((w[u][r].z >> 4) & M), d);
                    d = dot4_i8((int)a1.z, (int)(w[u][r].w & M), d);
                    d = dot4_i8((int)a1.w, (int)((w[u][r].w >> 4) & M), d);
                    acc[r] += (float)d * (as * __half2float(hs[u][r]));
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = wave_sum(acc[r]);
    if (row0 >= N) return;                                  // a tail wavefront without rows (after the workgroup's one barrier)

    // lane r finishes row r
    bool active = lane < R && row0 + lane < N;
    float val = acc[0];
#pragma unroll
    for (int r = 1; r < R; ++r) val = lane == r ? acc[r] : val;
    const int row = min(row0 + lane, N - 1);
    // Up the tree. Device-scope atomics only (they act at the device's coherence point); no device-scope fence: on this GPU
    // such a fence writes back and invalidates the whole L2 of the XCD, which costs more than the kernel. The exchange both
    // publishes this partial and fetches the sibling's, so nothing has to be ordered against anything else.
    int idx = s, base = 0;
    for (int width = S; width > 1; width >>= 1) {
        unsigned long long *word = meet + (size_t)(base + (idx >> 1)) * N + row;
        unsigned long long old = 0;
        if (active) old = __hip_atomic_exchange(word, (1ull << 32) | (unsigned long long)__float_as_uint(val), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool second = active && (old >> 32) != 0;
        if (second) {
            const float other = __uint_as_float((unsigned)old);
            val = (idx & 1) ? other + val : val + other;      // even slice + odd slice, whoever arrived second
            __hip_atomic_store(word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        active = second;
        if (!__builtin_amdgcn_ballot_w64(active)) return;
        base += width >> 1;
        idx >>= 1;
    }
    if (active) {
        const float out = alpha * val;
        c[row] = beta == 0.f ? out : out + beta * c[row];
    }
}


template <int DT, int R, int NT, int CPL>
void launch_s(aionhip_ctx *ctx, const aionhip_weight *w, float *c, const float *x, unsigned long long *meet, int groups, int kbs, int S,
              float alpha, float beta) {
    const dim3 grid((unsigned)groups * (unsigned)S), block(NT);
    // Bytes from one weight row to the next. Near 4, 8 or 32 KiB the slices alternate in dispatch order (measured over N =
    // 2048 ... 14336: 8 KiB from 4096 rows on, q8 8192 x 8192 19.4 -> 14.2 us, q4 8192 x 16384 20.2 -> 15.0; 4 KiB from 8192 rows
    // on, q4 8192 x 8192 9.3 -> 8.1; 32 KiB 3-25 %; 12, 16, 20, 24 KiB and every other pitch are 3-10 % better slice by slice).
    const size_t pitch = w->dtype == AIONHIP_Q8_0 ? w->k : w->k / 2;
    auto near = [&](size_t p) { return pitch + 128 >= p && pitch <= p + 128; };
    const int interleave = S > 1 && ((near(8192) && w->n >= 4096) || (near(4096) && w->n >= 8192) || near(32768)) ? 1 : 0;
    const size_t lds = (size_t)kbs * 40 + 16;
    const int n = (int)w->n, k = (int)w->k;
    const int per_pass = NT / 8;                            // quant blocks one pass of the workgroup prepares
    if (kbs <= per_pass) launch_k(ctx, gemv_ksplit_kernel<DT, R, NT, 1, CPL>, grid, block, lds, (const u32x4 *)w->qs, w->sc, c, x, meet, n, k, kbs, S, groups, interleave, alpha, beta);
    else if (kbs <= 2 * per_pass) launch_k(ctx, gemv_ksplit_kernel<DT, R, NT, 2, CPL>, grid, block, lds, (const u32x4 *)w->qs, w->sc, c, x, meet, n, k, kbs, S, groups, interleave, alpha, beta);
    else launch_k(ctx, gemv_ksplit_kernel<DT, R, NT, 4, CPL>, grid, block, lds, (const u32x4 *)w->qs, w->sc, c, x, meet, n, k, kbs, S, groups, interleave, alpha, beta);
}

template <int DT, int R, int NT>
void launch_c(aionhip_ctx *ctx, int cpl, const aionhip_weight *w, float *c, const float *x, unsigned long long *meet, int groups, int kbs,
              int S, float alpha, float beta) {
    if (cpl == 1) launch_s<DT, R, NT, 1>(ctx, w, c, x, meet, groups, kbs, S, alpha, beta);
    else if (cpl == 2) launch_s<DT, R, NT, 2>(ctx, w, c, x, meet, groups, kbs, S, alpha, beta);
    else launch_s<DT, R, NT, 4>(ctx, w, c, x, meet, groups, kbs, S, alpha, beta);
}

}  // namespace

bool gemv_ksplit_applies(const aionhip_ctx *ctx, const aionhip_weight *w, const float *x) {
    (void)ctx;
    // up to 8 slices of at most 256 16-byte chunks per row
    const size_t max_k = w->dtype == AIONHIP_Q8_0 ? 32768 : 65536;
    return w->k > FUSED_PAYS_K && w->k <= max_k && w->n <= 65536 && ((uintptr_t)x & 15) == 0;
}

int launch_gemv_ksplit(aionhip_ctx *ctx, const aionhip_weight *w, float *c, const float *x, float alpha, float beta) {
    const bool q8 = w->dtype == AIONHIP_Q8_0;
    const char *name = q8 ? "gemv_q8_ksplit" : "gemv_q4_ksplit";
    const int KB = (int)(w->k >> 5), N = (int)w->n;
    const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
    // Slices: the fewest (a power of two, at most 8) that leave a lane two 16-byte chunks per row, so that four rows per
    // wavefront are eight loads in flight per lane - all the wavefront will ever request, issued before anything is waited
    // for. Fewer rows per wavefront only when the weight is too small to give every CU four wavefronts.
    const int max_kbs = q8 ? 128 : 256, want_kbs = q8 ? 64 : 128;
    int S = 1, R = 4;
    while (S < KSPLIT_MAX_S && (KB + S - 1) / S > want_kbs) S *= 2;
    while (R > 1 && (long)((N + R - 1) / R) * S < (long)cus * 4) R >>= 1;
    const int NT = ((N + R - 1) / R >= 1024 || (KB + S - 1) / S > 128) ? 512 : 256;   // a 256-thread workgroup prepares at most 128 blocks
    const int kbs = (KB + S - 1) / S;
    const int nch = q8 ? 2 * kbs : kbs;
    const int cpl = nch <= 64 ? 1 : (nch <= 128 ? 2 : 4);
    const int wpb = NT / 64, groups = ((N + R - 1) / R + wpb - 1) / wpb;
    if ((S & (S - 1)) != 0 || S > KSPLIT_MAX_S || (long)kbs * (S - 1) >= KB || nch > 256 || kbs > NT / 2)
        return set_err(ctx, AIONHIP_UNSUPPORTED, "gemv ksplit: k = %zu does not cut into %d slices of at most %d blocks", w->k, S, max_kbs);
    const size_t need = (size_t)(S > 1 ? S - 1 : 1) * N * sizeof(unsigned long long);
    {
        // every meeting word starts empty and is left empty by the launch that used it
        const int rc = grow_work_buffer(ctx, &ctx->ksplit, &ctx->ksplit_bytes, need, true, "the K-split buffer");
        if (rc) return rc;
    }
    unsigned long long *meet = (unsigned long long *)ctx->ksplit;
    ProfScope scope(ctx, name);
#define KS_GO(DT_)                                                                                                 \
    do {                                                                                                           \
        if (NT == 1024) {                                                                                          \
            if (R == 1) launch_c<DT_, 1, 1024>(ctx, cpl, w, c, x, meet, groups, kbs, S, alpha, beta);  \
            else if (R == 2) launch_c<DT_, 2, 1024>(ctx, cpl, w, c, x, meet, groups, kbs, S, alpha, beta); \
            else launch_c<DT_, 4, 1024>(ctx, cpl, w, c, x, meet, groups, kbs, S, alpha, beta);         \
        } else if (NT == 512) {                                                                                    \
            if (R == 1) launch_c<DT_, 1, 512>(ctx, cpl, w, c, x, meet, groups, kbs, S, alpha, beta);   \
            else if (R == 2) launch_c<DT_, 2, 512>(ctx, cpl, w, c, x, meet, groups, kbs, S, alpha, beta); \
            else launch_c<DT_, 4, 512>(ctx, cpl, w, c, x, meet, groups, kbs, S, alpha, beta);          \
        } else {                                                                                                   \
            if (R == 1) launch_c<DT_, 1, 256>(ctx, cpl, w, c, x, meet, groups, kbs, S, alpha, beta);   \
            else if (R == 2) launch_c<DT_, 2, 256>(ctx, cpl, w, c, x, meet, groups, kbs, S, alpha, beta); \
            else launch_c<DT_, 4, 256>(ctx, cpl, w, c, x, meet, groups, kbs, S, alpha, beta);          \
        }                                                                                                          \
    } while (0)
    if (q8) KS_GO(AIONHIP_Q8_0);
    else KS_GO(AIONHIP_Q4_0);
#undef KS_GO
    LAUNCH_CHECK(ctx, name);
    return AIONHIP_OK;
}
