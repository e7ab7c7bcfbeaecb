// Attention step: grouped-query attention over token-major K/V with an interval window per query
// (aion graph/graph.zig:130-181,365-393; CPU executor cpu/exec/attention.zig:627-815,1347-1442).
//
// attn_flash_kernel - d_k = d_v in {64,128,256}, K/V f16 or bf16. Flash-style online softmax with
//   MFMA for both products, written in the transposed form so that no cross-lane shuffle of the
//   probabilities is needed:
//       S^T[keys x rows] = K_tile[keys x d] . Q^T[d x rows]          (A = K rows straight from HBM)
//       O^T[dv x rows]  += V_tile^T[dv x keys] . P^T[keys x rows]    (A = V^T gathered through LDS)
//   A wavefront owns 16 query rows (row = position-major, GQA head fastest, all sharing one K/V
//   head); each lane's accumulators, running max and sum belong to ONE query row, so the softmax
//   bookkeeping is per-lane scalar work. Two launch shapes:
//     split mode (few query rows: decode) - a workgroup is one 16-row tile x one key segment, its
//       eight wavefronts interleave 32-key tiles and merge through LDS; segments merge in
//       attn_merge_kernel (the flash-decoding split of cpu/exec/attention.zig:879-962).
//     per-wavefront mode - a workgroup is four 16-row tiles, each wavefront walks its own key range; used
//       for many query rows only when the hi+lo precise mode is on (see attn_prefill_kernel otherwise).
// attn_prefill_kernel (attention_prefill.hip) - many query rows: 128 rows per workgroup, K/V tiles shared through LDS,
//   32x32x16 MFMA (described at the kernel).
// attn_generic_kernel - any head size / f32 K,V: one wavefront per query row, scores staged in
//   global scratch. Slow; it exists so that every shape the op allows has a GPU path.
//
// Softmax uses exp2 on (s - m) * log2(e); aion's CPU path uses a 4th-order polynomial exp
// (cpu/kernels/fast_math.zig:79-92, rel. err 4e-5), so results agree to ~1e-4, not bitwise.
#include "attention_flash.h"

namespace {
using namespace attn;

// What the body does at its two seams when it is a kernel of its own: the queries are in global memory from the start,
// the output rows go to global memory as they are.
struct FlashKernelHooks {
    static constexpr bool Q_LATE = false;
    __device__ __forceinline__ void late_q(size_t, bool, f32x4 &, f32x4 &) {}
    __device__ __forceinline__ int new_key() { return -1; }
    __device__ __forceinline__ u32x4 new_k(int) { return u32x4{0u, 0u, 0u, 0u}; }
    __device__ __forceinline__ u32x4 new_v(int) { return u32x4{0u, 0u, 0u, 0u}; }
    __device__ __forceinline__ void store_out(float *out, size_t index, f32x4 v) { *(f32x4 *)(out + index) = v; }
};

template <int KV, int D, bool SPLIT, bool HILO, bool RING = false>
__global__ __launch_bounds__(SPLIT ? SPLIT_NW * 64 : 256) void attn_flash_kernel(AttnArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    FlashKernelHooks hooks;
    attn_flash_body<KV, D, SPLIT, HILO, RING>(a, lds, (int)blockIdx.x, (int)blockIdx.y, hooks);
}

// log-sum-exp merge of the key segments: one workgroup per (row tile, 16-wide dv slice, unit).
// Thread = (segment group of 4, row of 16, 4 consecutive dv): it folds every fourth segment with all
// of a round's loads in flight at once, then the four groups fold through LDS.
constexpr int MERGE_DV = 16, MERGE_SG = 4, MERGE_UNROLL = 8;
template <int D>
__global__ __launch_bounds__(256) void attn_merge_kernel(AttnArgs a) {
    constexpr int WSTRIDE = 16 * D + 32;
    constexpr int SLICES = D / MERGE_DV;
    __shared__ float s_m[MERGE_SG][16][4], s_l[MERGE_SG][16][4];
    __shared__ __attribute__((aligned(16))) float s_o[MERGE_SG][16][MERGE_DV];
    const int unit = blockIdx.y, rt = blockIdx.x / SLICES, slice = blockIdx.x % SLICES;
    const int b = unit / a.Hkv, hk = unit % a.Hkv;
    const int tid = threadIdx.x, q4 = tid & 3, row = (tid >> 2) & 15, sg = tid >> 6;
    const float *base = a.partial + (size_t)(unit * a.row_tiles + rt) * a.nseg * WSTRIDE;
    const int dv = slice * MERGE_DV + q4 * 4;
    // padding rows of the last tile were never stored: their threads read the tile's last real row instead (the same lines
    // its own threads fetch) and drop the result below
    const int row_ld = min(row, min(16, a.rows_total - rt * 16) - 1);
    float m_loc = -INFINITY, l_loc = 0.f;
    f32x4 o_loc = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int s0 = sg; s0 < a.nseg; s0 += MERGE_SG * MERGE_UNROLL) {
        float ms[MERGE_UNROLL], ls[MERGE_UNROLL];
        f32x4 os[MERGE_UNROLL];
#pragma unroll
        for (int u = 0; u < MERGE_UNROLL; ++u) {
            const int sidx = min(s0 + u * MERGE_SG, a.nseg - 1);      // clamped: every load is unconditional
            const float *p = base + (size_t)sidx * WSTRIDE;
            ms[u] = p[16 * D + row_ld];
            ls[u] = p[16 * D + 16 + row_ld];
            os[u] = *(const f32x4 *)(p + row_ld * D + dv);
        }
        float m_new = m_loc;
#pragma unroll
        for (int u = 0; u < MERGE_UNROLL; ++u)
            if (s0 + u * MERGE_SG < a.nseg) m_new = fmaxf(m_new, ms[u]);
        if (m_new > -INFINITY) {
            const float f0 = m_loc > -INFINITY ? exp2f((m_loc - m_new) * LOG2E) : 0.f;
            o_loc *= f0;
            l_loc *= f0;
#pragma unroll
            for (int u = 0; u < MERGE_UNROLL; ++u) {
                const bool live = s0 + u * MERGE_SG < a.nseg && ms[u] > -INFINITY;
                const float f = live ? exp2f((ms[u] - m_new) * LOG2E) : 0.f;
                o_loc += os[u] * f;
                l_loc += ls[u] * f;
            }
            m_loc = m_new;
        }
    }
    s_m[sg][row][q4] = m_loc;
    s_l[sg][row][q4] = l_loc;
    *(f32x4 *)&s_o[sg][row][q4 * 4] = o_loc;
    __syncthreads();
    if (sg == 0) {
        float m_all = -INFINITY;
#pragma unroll
        for (int g2 = 0; g2 < MERGE_SG; ++g2) m_all = fmaxf(m_all, s_m[g2][row][q4]);
        f32x4 o = f32x4{0.f, 0.f, 0.f, 0.f};
        float l_all = 0.f;
#pragma unroll
        for (int g2 = 0; g2 < MERGE_SG; ++g2) {
            const float mg = s_m[g2][row][q4];
            const float f = mg > -INFINITY ? exp2f((mg - m_all) * LOG2E) : 0.f;
            o += *(const f32x4 *)&s_o[g2][row][q4 * 4] * f;
            l_all += s_l[g2][row][q4] * f;
        }
        const int rr = rt * 16 + row;
        if (rr < a.rows_total) {
            const int l2 = rr / a.groups, g3 = rr % a.groups;
            const float inv = l_all > 0.f ? 1.f / l_all : 0.f;
            *(f32x4 *)(a.out + (((size_t)b * a.L + l2) * a.Hq + hk * a.groups + g3) * D + dv) = o * inv;
        }
    }
}

// One wavefront per query row; any head sizes and element types. scores: [rows][T] f32 scratch.
__global__ __launch_bounds__(256) void attn_generic_kernel(AttnArgs a, int d_k, int d_v, float *scores) {
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const size_t total_rows = (size_t)a.B * a.L * a.Hq;
    if (row >= total_rows) return;
    const int hq = (int)(row % a.Hq);
    const int li = (int)((row / a.Hq) % a.L);
    const int b = (int)(row / ((size_t)a.Hq * a.L));
    const int hk = hq / a.groups;
    const int kv_end = clip_kv_end(a.ring, a.T, a.kv_lengths ? a.kv_lengths[b] : a.T);
    const int pos = a.positions ? a.positions[(size_t)b * a.L + li] : li;
    int lo, hi;
    window_keys(a.win_left, a.win_right, a.win_chunk, max(pos, 0), kv_end, lo, hi);
    clip_to_ring(a.ring, kv_end, lo, hi);
    float *o = a.out + row * d_v;
    if (hi <= lo) {
        for (int j = lane; j < d_v; j += 64) o[j] = 0.f;
        return;
    }
    float *sc = scores + row * a.T;
    const size_t qb = row * d_k;
    float mx = -INFINITY;
    // scores are kept at the key's physical row: a ring's visible keys span at most T steps
    for (int t = lo + lane; t < hi; t += 64) {
        const int tp = phys_key(a.ring, t);
        const size_t kb = (((size_t)b * a.T + tp) * a.Hkv + hk) * d_k;
        float d = 0.f;
        for (int j = 0; j < d_k; ++j) d += (load_scalar(a.q, a.q_dtype, qb + j) * a.scale) * load_scalar(a.k, a.kv_dtype, kb + j);
        if (a.soft_cap > 0.f) d = a.soft_cap * tanhf(d / a.soft_cap);
        sc[tp] = d;
        mx = fmaxf(mx, d);
    }
    mx = wave_max(mx);
    float sum = 0.f;
    for (int t = lo + lane; t < hi; t += 64) {
        const int tp = phys_key(a.ring, t);
        const float p = exp2f((sc[tp] - mx) * LOG2E);
        sc[tp] = p;
        sum += p;
    }
    sum = wave_sum(sum);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    const float inv = 1.f / sum;
    for (int j = lane; j < d_v; j += 64) {
        float acc = 0.f;
        for (int t = lo; t < hi; ++t) {
            const int tp = phys_key(a.ring, t);
            acc += sc[tp] * load_scalar(a.v, a.kv_dtype, (((size_t)b * a.T + tp) * a.Hkv + hk) * d_v + j);
        }
        o[j] = acc * inv;
    }
}

template <int KV, int D, bool HILO, bool RING = false>
int launch_flash(aionhip_ctx *ctx, AttnArgs &a) {
    using Cfg = FlashCfg<D, 4>;
    using SplitCfg = FlashCfg<D, SPLIT_NW>;
    const int units = a.B * a.Hkv;
    // Few query rows, or so few 128-row prefill workgroups that they would occupy under a quarter of the CUs
    // (measured: one batch, one kv head, up to ~1024 positions x 8 heads): 16-row tiles spread the K/V reads
    // over many CUs, which outweighs re-reading K/V per row tile from L2.
    const int cus0 = ctx->cu_count > 0 ? ctx->cu_count : 256;
    // (the smaller the head, the longer the 16-row kernel stays ahead: per key it re-reads less. Crossovers measured over
    // five head layouts x L = 128 .. 2048: about 80 / 40 / 32 workgroups of the 128-row kernel at head size 64 / 128 / 256)
    const long pf_wgs = (long)units * ((a.rows_total + PF_ROWS - 1) / PF_ROWS);
    const long pf_min = D <= 64 ? (long)cus0 * 5 / (2 * PF_FLASH_BELOW) : D <= 128 ? (long)cus0 * 5 / (4 * PF_FLASH_BELOW) : (long)cus0 / PF_FLASH_BELOW;
    bool split = a.rows_total <= 64 || (!HILO && pf_wgs <= pf_min) ||
                 (!HILO && !prefill_takes(a, D));      // e.g. a softmax scale that is not positive: the 16-row kernel takes any
    // A chunk of queries over a cache at least four times its length (chunked prompts, speculative batches): the crossover
    // above was measured on prompts over their own keys, where few rows mean few keys. Here the keys dominate, and the 128-row
    // kernel, which can cut them into up to 16 segments, is weighed against the 16-row kernel by what both measured over
    // 1 ... 1024 queries x 1024 ... 16384 keys at head sizes 128 and 256: the 16-row kernel 13 us + 0.56 us per 32-key tile a
    // workgroup walks (head size 256; in proportion below), the 128-row kernel 16 us + 1.9 us per 64-key tile (1.2 at head
    // size 128, 0.85 at 64; 0.7 of that while half the CUs stay free). 8 heads x 256, 256 queries over 16384 keys: 159 -> 46 us.
    if (!HILO && a.rows_total > 64 && pf_wgs <= pf_min && prefill_takes(a, D) && (long)a.T >= 4L * a.L && a.win_left >= (unsigned)a.T) {
        const float ds = (float)D / 256.f;
        const long wgs16 = (long)units * a.row_tiles;
        const int tiles32 = (a.T + TILE_KEYS - 1) / TILE_KEYS;
        const long nseg_s = max(1L, min((long)cus0 / max(wgs16, 1L), (long)(tiles32 + SPLIT_NW - 1) / SPLIT_NW));
        const long rounds_s = (wgs16 * nseg_s + cus0 - 1) / cus0;
        const float split_us = (nseg_s > 1 ? 13.f : 10.f) + (float)((tiles32 + nseg_s - 1) / nseg_s) * 0.56f * ds * (float)rounds_s;
        const int tiles64 = (a.T + PF_TK - 1) / PF_TK;
        const long nseg_p = max(1L, min(min((long)cus0 / max(pf_wgs, 1L), (long)tiles64 / (D > 128 ? 4 : 8)), 16L));
        const long rounds_p = (pf_wgs * nseg_p + cus0 - 1) / cus0;
        const float per_tile = (0.5f + 1.4f * ds) * (pf_wgs * nseg_p * 2 <= cus0 ? 0.7f : 1.f);
        const float prefill_us = (nseg_p > 1 ? 16.f : 12.f) + (float)((tiles64 + nseg_p - 1) / nseg_p) * per_tile * (float)rounds_p;
        if (prefill_us < split_us) split = false;
    }
    if (split) {
        // key segments: one 32-key tile per wavefront while that leaves the device under-filled,
        // more tiles per wavefront beyond one workgroup per CU (its LDS tiles fill a CU)
        const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
        const int tiles = (a.T + TILE_KEYS - 1) / TILE_KEYS;
        // (as many segments as keep the workgroups within one per CU: a second, partial round of workgroups plus the merge
        // launch costs more than CUs left idle - 192 row tiles in two segments each took 26 us, in one 13)
        int nseg = cus / (units * a.row_tiles);
        nseg = max(1, min(nseg, (tiles + SPLIT_NW - 1) / SPLIT_NW));
        nseg = min(nseg, 256);
        a.nseg = nseg;
        if (nseg > 1) {
            const size_t bytes = (size_t)units * a.row_tiles * nseg * (16 * D + 32) * sizeof(float);
            int rc = ensure_scratch2(ctx, bytes);
            if (rc) return rc;
            a.partial = (float *)ctx->scratch2;
        }
        static bool attr_split = false;   // per kernel instantiation
        if (!attr_split) {
            HIP_TRY(ctx, hipFuncSetAttribute((const void *)attn_flash_kernel<KV, D, true, HILO, RING>, hipFuncAttributeMaxDynamicSharedMemorySize, SplitCfg::LDS_BYTES));
            attr_split = true;
        }
        {
            ProfScope scope(ctx, "attn_flash_split");
            launch_k(ctx, attn_flash_kernel<KV, D, true, HILO, RING>, dim3((unsigned)(a.row_tiles * nseg), (unsigned)units), dim3(SPLIT_NW * 64), SplitCfg::LDS_BYTES, a);
        }
        if (nseg > 1) {
            ProfScope scope(ctx, "attn_merge");
            launch_k(ctx, attn_merge_kernel<D>, dim3((unsigned)(a.row_tiles * (D / MERGE_DV)), (unsigned)units), dim3(256), 0, a);
        }
        LAUNCH_CHECK(ctx, "attn_flash_split");
    } else if (!HILO) {
        return launch_prefill(ctx, a, D);
    } else {
        a.nseg = 1;
        static bool attr_prefill = false;
        if (!attr_prefill) {
            HIP_TRY(ctx, hipFuncSetAttribute((const void *)attn_flash_kernel<KV, D, false, HILO>, hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES));
            attr_prefill = true;
        }
        ProfScope scope(ctx, "attn_flash_prefill");
        launch_k(ctx, attn_flash_kernel<KV, D, false, HILO>, dim3((unsigned)((a.row_tiles + 3) / 4), (unsigned)units), dim3(256), Cfg::LDS_BYTES, a);
        LAUNCH_CHECK(ctx, "attn_flash_prefill");
    }
    return AIONHIP_OK;
}

template <int KV>
int launch_flash_d(aionhip_ctx *ctx, AttnArgs &a, int d) {
    const bool hilo = a.q_dtype == AIONHIP_F32 && ctx->attn_precise;
    if (a.ring) {       // rolling caches: the plain instances only (precise mode and soft cap take the generic kernel)
        if (d == 64) return launch_flash<KV, 64, false, true>(ctx, a);
        if (d == 128) return launch_flash<KV, 128, false, true>(ctx, a);
        return launch_flash<KV, 256, false, true>(ctx, a);
    }
    if (d == 64) return hilo ? launch_flash<KV, 64, true>(ctx, a) : launch_flash<KV, 64, false>(ctx, a);
    if (d == 128) return hilo ? launch_flash<KV, 128, true>(ctx, a) : launch_flash<KV, 128, false>(ctx, a);
    return hilo ? launch_flash<KV, 256, true>(ctx, a) : launch_flash<KV, 256, false>(ctx, a);
}

bool dtype_ok(int d) { return d == AIONHIP_F32 || d == AIONHIP_F16 || d == AIONHIP_BF16; }

}  // namespace

extern "C" int aionhip_step_attention(aionhip_ctx *ctx, const aionhip_attention *p) {
    if (!ctx || !p) return AIONHIP_INVALID_ARGUMENT;
    if (!p->out || !p->q || !p->k || !p->v) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "attention: null operand");
    if (!dtype_ok(p->q_dtype) || !dtype_ok(p->kv_dtype)) return set_err(ctx, AIONHIP_UNSUPPORTED, "attention: q/kv dtype must be f32, f16 or bf16");
    if (p->h_kv == 0 || p->h_q == 0 || p->h_q % p->h_kv != 0) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "attention: h_q %zu is not a multiple of h_kv %zu", p->h_q, p->h_kv);
    if (p->d_k == 0 || p->d_v == 0) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "attention: zero head size");
    if (p->batch == 0 || p->l_q == 0) return AIONHIP_OK;
    const size_t lim = 0x7FFFFFFF;
    if (p->batch > lim || p->l_q > lim || p->t_kv > lim || p->h_q > 65535 || p->d_k > 65535 || p->d_v > 65535 ||
        p->batch * p->h_kv > 65535 || p->l_q * (p->h_q / p->h_kv) > lim)
        return set_err(ctx, AIONHIP_UNSUPPORTED, "attention: dimension too large");

    AttnArgs a{};
    a.q = (const void *)(uintptr_t)p->q;
    a.k = (const void *)(uintptr_t)p->k;
    a.v = (const void *)(uintptr_t)p->v;
    a.out = (float *)(uintptr_t)p->out;
    a.positions = (const int *)(uintptr_t)p->query_positions;
    a.kv_lengths = (const int *)(uintptr_t)p->kv_lengths;
    a.B = (int)p->batch; a.L = (int)p->l_q; a.T = (int)p->t_kv; a.Hq = (int)p->h_q; a.Hkv = (int)p->h_kv;
    a.groups = a.Hq / a.Hkv;
    a.rows_total = a.L * a.groups;
    a.row_tiles = (a.rows_total + 15) / 16;
    a.nseg = 1;
    a.q_dtype = p->q_dtype; a.kv_dtype = p->kv_dtype;
    a.scale = p->scale; a.soft_cap = p->attn_logits_soft_cap;
    a.win_left = p->window_left; a.win_right = p->window_right; a.win_chunk = p->window_chunk;
    a.ring = p->rolling ? a.T : 0;

    if (a.T == 0) {
        // no keys at all: every interval is empty -> zeros (cpu/exec/attention.zig:787-815)
        return aionhip_memset(ctx, p->out, 0, 0, p->batch * p->l_q * p->h_q * p->d_v * sizeof(float));
    }

    const bool flash = p->d_k == p->d_v && (p->d_k == 64 || p->d_k == 128 || p->d_k == 256) &&
                       (p->kv_dtype == AIONHIP_F16 || p->kv_dtype == AIONHIP_BF16) &&
                       ((p->k | p->v | p->out) & 15) == 0 &&
                       // a ring shorter than a key tile, or a ring in precise / soft-cap mode: generic kernel
                       (!a.ring || (a.T >= PF_TK && !(a.q_dtype == AIONHIP_F32 && ctx->attn_precise) && a.soft_cap <= 0.f));
    if (flash) {
        if (p->kv_dtype == AIONHIP_F16) return launch_flash_d<AIONHIP_F16>(ctx, a, (int)p->d_k);
        return launch_flash_d<AIONHIP_BF16>(ctx, a, (int)p->d_k);
    }
    const size_t rows = p->batch * p->l_q * p->h_q;
    int rc = ensure_scratch2(ctx, rows * p->t_kv * sizeof(float));
    if (rc) return rc;
    ProfScope scope(ctx, "attn_generic");
    launch_k(ctx, attn_generic_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, a, (int)p->d_k, (int)p->d_v, (float *)ctx->scratch2);
    LAUNCH_CHECK(ctx, "attn_generic");
    return AIONHIP_OK;
}
