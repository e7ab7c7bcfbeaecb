// Prefill attention: many query rows per K/V head (aion graph/graph.zig:130-181,365-393; CPU executor
// cpu/exec/attention.zig:627-815). attn_prefill_kernel and the merge of its key segments, with their launcher.
//
// This file is compiled with MFMA results in vector registers (-mllvm -amdgpu-mfma-vgpr-form): the scores of a key
// tile feed the softmax straight from the registers the MFMA wrote, and the rescale of the output accumulators is a
// plain multiply. The other attention kernels (attention.hip) keep the compiler's default register form.
#include "attention_common.h"

namespace {
using namespace attn;

// ------------------------------------------------------------------------------------------------
// attn_prefill_kernel - many query rows (prefill), q already in the K/V element type or f32 (rounded).
//   A workgroup owns 128 query rows of one (batch, kv head) - position-major, GQA head fastest - and
//   walks the 32-key tiles of the union of their intervals once; K and V tiles are loaded by the whole
//   workgroup and shared through LDS (double-buffered, one barrier per tile), so a K/V byte fetched
//   from L2 feeds 128 rows instead of 16. Each wavefront owns 32 rows and works in the transposed
//   form on v_mfma_f32_32x32x16:
//       S^T[32 keys x 32 rows]  = K_tile[32 x D] . Q^T[D x 32]       A = K rows from LDS (16 B reads)
//       O^T[D x 32 rows]       += V^T[D x 32 keys] . P^T[32 x 32]    A = V^T rows from LDS (8 B reads)
//   so every accumulator, the running max and the running sum of a lane belong to ONE query row.
//   V is transposed once per tile by the loading threads (two keys packed per 32-bit store into
//   V^T[dv][key], row stride 72 B: stores and operand reads are bank-conflict-free); the k index of
//   the second product is permuted (slot s of lane half h <-> key (s/4)*8 + 4h + s%4 of a 16-key step)
//   so that the probabilities feed the MFMA straight from the S accumulators without a shuffle.
constexpr int PF_VROW = 136;
constexpr float PF_LAZY = 8.f;
#ifndef PF_AHEAD
#define PF_AHEAD 3
#endif
#ifndef PF_SEG_TILES
#define PF_SEG_TILES 4     // fewest 64-key tiles a key segment of the prefill kernel is worth
#endif
#ifndef PF_TWO_SEG_BELOW_TENTHS
#define PF_TWO_SEG_BELOW_TENTHS 12   // row tiles up to 1.2 x the CUs: two key segments per tile
#endif
#ifndef PF_PIPE_D
#define PF_PIPE_D 128      // head sizes from here on run the software-pipelined tile loop
#endif
using f32x16 = __attribute__((ext_vector_type(16))) float;
// wait states between the last MFMA of a score tile and the hand-written vector read of its results (see unit 0 of the tile loop)
constexpr int PF_SCORE_MFMA_PASSES = 8;                        // v_mfma_f32_32x32x16_{f16,bf16} on gfx950
constexpr int PF_SCORE_WAIT = PF_SCORE_MFMA_PASSES + 4 + 2;    // required + margin
static_assert(PF_SCORE_WAIT > 8 && PF_SCORE_WAIT <= 16, "two s_nop instructions cover 9..16 wait states");

using v4s16 = __attribute__((ext_vector_type(4))) short;
typedef __attribute__((address_space(3))) v4s16 lds_v4s16;
// Softmax units of the pipelined prefill loop (46 of them, see there) dealt out behind the nm MFMAs of the product by
// issue cost: unit u goes behind MFMA k when the cost of units 0..u first exceeds k/nm of the total. Returns the first
// unit that does NOT go behind MFMAs 0..k-1.
constexpr int pf_unit_cost(int u) { return u < 8 ? 2 : (u == 8 ? 12 : (u < 41 ? 5 : (u < 45 ? 8 : 4))); }
constexpr int pf_unit_end(int k, int nm) {
    int total = 0;
    for (int u = 0; u < 46; ++u) total += pf_unit_cost(u);
    if (k >= nm) return 46;
    int run = 0, u = 0;
    // units whose cumulative cost stays within k/nm of the total
    while (u < 46 && (run + pf_unit_cost(u)) * nm <= total * k) run += pf_unit_cost(u++);
    return u;
}
// A key segment's partial result for one 16-row tile: [16][D] accumulators, then the rows' reference maxima and sums.
// Over a bf16 cache the accumulators are stored as f16 (the probabilities of the second product carry 8 bits, the f16
// accumulators 11), each row scaled by a power of two so that any bf16 value range fits, with that scale as a third
// per-row float; the values of a row stand in the order the lanes hold them (position j*32 + h*16 + q*4 + i holds dv
// j*32 + q*8 + h*4 + i), 32 contiguous bytes per lane and dv tile. Half the bytes written by the tile kernel and read
// by the merge: both are bound by the bytes they move (the workgroups of a round all store at the same time).
constexpr bool pf_half_partials(int kv) { return kv == AIONHIP_BF16; }
constexpr int pf_partial_bytes(int d, bool half) { return half ? 32 * d + 192 : 64 * d + 128; }

template <int D>
struct PrefillCfg {
    static constexpr int KROW = D * 2;                              // unpadded (filled by LDS-writing loads), chunk slots swizzled
    static constexpr int K_BYTES = PF_TK * KROW;
    static constexpr int V_BYTES = D * PF_VROW;
    static constexpr int STAGE = K_BYTES + V_BYTES;
    static constexpr int LDS_BYTES = 2 * STAGE + 64;
};

// acc + lo half + hi half of a packed pair of f16 / bf16 values
template <int KV>
__device__ __forceinline__ float dot2_ones(unsigned pair, float acc) {
    using f16x2 = __attribute__((ext_vector_type(2))) _Float16;
    using bf16x2 = __attribute__((ext_vector_type(2))) __bf16;
    if (KV == AIONHIP_F16) return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, pair), f16x2{(_Float16)1.f, (_Float16)1.f}, acc, false);
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pair), __builtin_bit_cast(bf16x2, 0x3F803F80u), acc, false);
}

template <int KV>
__device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
    if (KV == AIONHIP_F16)
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

template <int KV, int D, bool CAP, bool RING = false>
__global__ __launch_bounds__(256) void attn_prefill_kernel(AttnArgs a) {
    const int ring = RING ? a.ring : 0;
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
    using Cfg = PrefillCfg<D>;
    constexpr int KK = D / 16;          // k-steps of the first product
    constexpr int NJ = D / 32;          // 32-wide dv tiles of the second product
    constexpr int CPK = D / 8;          // 16-byte chunks per key row
    constexpr int NKI = PF_TK * Cfg::KROW / 1024 / 4;   // K loads (1 KiB each) per wavefront per tile
    constexpr int KEYS_PER_KI = 1024 / Cfg::KROW;       // keys covered by one K load
    (void)KEYS_PER_KI;                                  // (the loads are in the device pass only)
    constexpr int V_ITEMS = (PF_TK / 2) * CPK;          // V (key pair, chunk) items per tile
    constexpr int NVL = V_ITEMS / 256;
    static_assert(NKI >= 1 && NVL >= 1, "head size below 64 is not handled here");

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l31 = lane & 31, lh = lane >> 5;
    const int unit = blockIdx.y, b = unit / a.Hkv, hk = unit % a.Hkv;

    // ---- this lane's query row (lanes l and l+32 share it)
    // row tiles in descending order: under a causal mask the last rows see the most keys, and workgroups are
    // dispatched in index order - the long ones start first and the short ones fill the gaps at the end
    const int r = ((int)gridDim.x - 1 - (int)blockIdx.x) * PF_ROWS + wave * 32 + l31;
    const bool row_ok = r < a.rows_total;
    const int li = row_ok ? r / a.groups : 0, gi = row_ok ? r % a.groups : 0;
    const int hq = hk * a.groups + gi;
    const int kv_end_raw = a.kv_lengths ? a.kv_lengths[b] : a.T;
    const int pos_raw = (row_ok && a.positions) ? a.positions[(size_t)b * a.L + li] : li;
    const size_t qbase = (((size_t)b * a.L + li) * a.Hq + hq) * D;

    // Q^T operand: lane (row l31, half lh) holds d = 16*kk + 8*lh .. +7 for every kk
    u32x4 qf[KK];
    if (a.q_dtype == KV) {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) qf[kk] = *(const u32x4 *)((const unsigned short *)a.q + qbase + kk * 16 + lh * 8);
    } else if (a.q_dtype == AIONHIP_F32 && (((uintptr_t)a.q) & 15) == 0) {
        // f32 queries (aion's decode graphs: f32 q over an f16 cache): 16-byte loads, all requested before the first is converted
        f32x4 x0[KK], x1[KK];
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const f32x4 *qp = (const f32x4 *)((const float *)a.q + qbase + kk * 16 + lh * 8);
            x0[kk] = qp[0];
            x1[kk] = qp[1];
        }
#pragma unroll
        for (int kk = 0; kk < KK; ++kk)
            qf[kk] = u32x4{pack2<KV>(x0[kk].x, x0[kk].y), pack2<KV>(x0[kk].z, x0[kk].w), pack2<KV>(x1[kk].x, x1[kk].y), pack2<KV>(x1[kk].z, x1[kk].w)};
    } else {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            float x[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) x[j] = load_scalar(a.q, a.q_dtype, qbase + kk * 16 + lh * 8 + j);
            qf[kk] = u32x4{pack2<KV>(x[0], x[1]), pack2<KV>(x[2], x[3]), pack2<KV>(x[4], x[5]), pack2<KV>(x[6], x[7])};
        }
    }
    if (!row_ok) {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) qf[kk] = u32x4{0u, 0u, 0u, 0u};
    }

    const int kv_end = clip_kv_end(ring, a.T, kv_end_raw);
    int lo = 0, hi = 0;
    if (row_ok) {
        window_keys(a.win_left, a.win_right, a.win_chunk, max(pos_raw, 0), kv_end, lo, hi);
        clip_to_ring(ring, kv_end, lo, hi);
    }
    const bool live = hi > lo;
    // wavefront: union (which tiles it computes) and intersection (which tiles need no mask)
    const int w_lo = wave_min_i(live ? lo : INT_MAX), w_hi = wave_max_i(live ? hi : 0);
    const int w_lo_max = wave_max_i(live ? lo : INT_MAX), w_hi_min = wave_min_i(live ? hi : 0);
    // workgroup union through LDS
    int *s_rng = (int *)(lds + 2 * Cfg::STAGE);
    if (lane == 0) { s_rng[wave] = w_lo; s_rng[4 + wave] = w_hi; }
    __syncthreads();
    const int g_lo = min(min(s_rng[0], s_rng[1]), min(s_rng[2], s_rng[3]));
    const int g_hi = max(max(s_rng[4], s_rng[5]), max(s_rng[6], s_rng[7]));
    // key segments (a.nseg > 1: few row tiles on many CUs): workgroup z takes the z-th part of the union's tiles and
    // leaves its unnormalized accumulators, reference maximum and sum in the partial buffer for attn_merge_kernel
    const int nseg = a.nseg, seg = blockIdx.z;
    int t_begin = g_lo / PF_TK, t_end = (g_hi + PF_TK - 1) / PF_TK;
    bool nothing = g_hi <= g_lo;
    if (nseg > 1 && !nothing) {
        const int per = (t_end - t_begin + nseg - 1) / nseg;
        t_begin += seg * per;
        t_end = min(t_end, t_begin + per);
        nothing = t_begin >= t_end;
    }
    constexpr bool HP = pf_half_partials(KV);
    constexpr int PART_BYTES = pf_partial_bytes(D, HP);
    unsigned char *part = nullptr;
    if (nseg > 1) part = (unsigned char *)a.partial + ((size_t)(unit * a.row_tiles + (r >> 4)) * nseg + seg) * PART_BYTES;
    float *part_stats = (float *)(part + (HP ? 32 * D : 64 * D));          // [16] maxima, [16] sums, (f16 form) [16] scales
    if (nothing) {                                      // nothing visible to any row: zeros / an empty partial
        if (row_ok) {
            if (HP && nseg > 1) {
                unsigned char *o = part + (r & 15) * (D * 2) + lh * D;
                for (int d = 0; d < D; d += 16) *(u32x4 *)(o + d) = u32x4{0u, 0u, 0u, 0u};
            } else {
                float *o = nseg > 1 ? (float *)part + (r & 15) * D : a.out + qbase;
                for (int d = lh * (D / 2); d < (lh + 1) * (D / 2); d += 4) *(f32x4 *)(o + d) = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            if (nseg > 1 && lh == 0) {
                part_stats[r & 15] = -INFINITY;
                part_stats[16 + (r & 15)] = 0.f;
                if (HP) part_stats[32 + (r & 15)] = 1.f;
            }
        }
        return;
    }

    const unsigned short *kp = (const unsigned short *)a.k;
    const unsigned short *vp = (const unsigned short *)a.v;
    const size_t kv_row = (size_t)a.Hkv * D;
    const size_t kv_base = ((size_t)b * a.T * a.Hkv + hk) * D;
    const int key_clamp_hi = g_hi - 1;

    // ---- cooperative tile loads. K: global -> LDS directly, 1 KiB per instruction; the 16-byte chunk c of key k
    // sits at slot c ^ swz(k), swz = k & 15 (k >> 1 & 7 for 128-byte rows), so that the 16 consecutive keys of
    // an operand read hit 16 distinct bank groups. V: registers now, transposed stores after this tile's MFMAs.
    // Keys outside the union are read from a clamped in-range key (masked scores / exact-zero probabilities).
    const int k_key_in = (lane * 16) / Cfg::KROW, k_slot = ((lane * 16) % Cfg::KROW) / 16;
    (void)k_key_in; (void)k_slot;
    auto load_k = [&](int t, unsigned char *st) {
#if defined(__HIP_DEVICE_COMPILE__)   // the builtin exists in the device pass only
        const int key0 = t * PF_TK;
        const TileMap tm(ring, key0);
#pragma unroll
        for (int i = 0; i < NKI; ++i) {
            const int key = (wave * NKI + i) * KEYS_PER_KI + k_key_in;
            const int swz = CPK >= 16 ? (key & 15) : ((key >> 1) & 7);
            const int kabs = tm.row(min(max(key0 + key, g_lo), key_clamp_hi));
            __builtin_amdgcn_global_load_lds(kp + kv_base + (size_t)kabs * kv_row + (k_slot ^ swz) * 8,
                                             (lds_void *)(st + (wave * NKI + i) * 1024), 16, 0, 0);
        }
#endif
    };
    u32x4 vreg[NVL][2];
    auto load_v = [&](int t) {
        const int key0 = t * PF_TK;
        const TileMap tm(ring, key0);
#pragma unroll
        for (int i = 0; i < NVL; ++i) {
            const int id = tid + 256 * i, pair = (id & 15) + 16 * (id / (16 * CPK)), c = (id >> 4) % CPK;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int kabs = tm.row(min(max(key0 + pair * 2 + h, g_lo), key_clamp_hi));
                vreg[i][h] = *(const u32x4 *)(vp + kv_base + (size_t)kabs * kv_row + c * 8);
            }
        }
    };
    auto store_v = [&](unsigned char *st) {
#pragma unroll
        for (int i = 0; i < NVL; ++i) {
            const int id = tid + 256 * i, pair = (id & 15) + 16 * (id / (16 * CPK)), c = (id >> 4) % CPK;
            unsigned char *vt = st + Cfg::K_BYTES + (c * 8) * PF_VROW + pair * 4;
            const u32x4 x = vreg[i][0], y = vreg[i][1];
            const unsigned xs[4] = {x.x, x.y, x.z, x.w}, ys[4] = {y.x, y.y, y.z, y.w};
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                *(unsigned *)(vt + (2 * w) * PF_VROW) = (xs[w] & 0xFFFFu) | (ys[w] << 16);
                *(unsigned *)(vt + (2 * w + 1) * PF_VROW) = (xs[w] >> 16) | (ys[w] & 0xFFFF0000u);
            }
        }
    };

    f32x16 acc[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[j][i] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;
    const float cap_inv = CAP ? 1.f / a.soft_cap : 0.f;

    if constexpr (D < PF_PIPE_D) {
    load_k(t_begin, lds);
    load_v(t_begin);
    store_v(lds);
    __syncthreads();                                               // also waits for the K loads (fence)

    // operand addresses: K row (kb*32 + l31) at slot (2*kk + lh) ^ swz(row); V^T row (j*32 + l31), keys of step s2
    const int k_swz = CPK >= 16 ? (l31 & 15) : ((l31 >> 1) & 7);
    const int k_row = l31 * Cfg::KROW;
    const int v_off = Cfg::K_BYTES + l31 * PF_VROW + lh * 8;        // + j * 32 rows + s2 * 32 bytes (+16 for the second 4 keys)
    for (int t = t_begin; t < t_end; ++t) {
        const unsigned char *st = lds + ((t - t_begin) & 1) * Cfg::STAGE;
        unsigned char *nx = lds + ((t - t_begin + 1) & 1) * Cfg::STAGE;
        const bool more = t + 1 < t_end;
        if (more) {
            load_k(t + 1, nx);
            load_v(t + 1);
        }
        const int key0 = t * PF_TK;
        // Every wavefront computes every tile of the workgroup's union, also one that none of its own rows sees
        // (all of its scores are then masked and it adds exact zeros): the wavefronts meet at the barrier below
        // anyway.
        {
            // -- S^T = K . Q^T for the two 32-key halves (two independent accumulation chains)
            f32x16 s[2];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int i = 0; i < 16; ++i) s[kb][i] = 0.f;
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                const int slot = ((2 * kk + lh) ^ k_swz) * 16;
                const u32x4 k0 = *(const u32x4 *)(st + k_row + slot);
                const u32x4 k1 = *(const u32x4 *)(st + 32 * Cfg::KROW + k_row + slot);
                s[0] = mfma32<KV>(k0, qf[kk], s[0]);
                s[1] = mfma32<KV>(k1, qf[kk], s[1]);
            }
            // issue order: the LDS reads run PF_AHEAD k-steps ahead of the MFMAs that consume them (left alone the
            // compiler issues each read right before its MFMA, which then waits out the whole LDS latency)
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * PF_AHEAD, 0);
#pragma unroll
            for (int kk = 0; kk < KK - PF_AHEAD; ++kk) {
                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, 2 * PF_AHEAD, 0);
            // -- lane holds keys key0 + kb*32 + (i/4)*8 + lh*4 + i%4 of row l31
            float x[32];
            const bool full = key0 >= w_lo_max && key0 + PF_TK <= w_hi_min;   // every key visible to every row
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                float v = s[i >> 4][i & 15] * a.scale;
                if (CAP) v = a.soft_cap * tanhf(v * cap_inv);
                x[i] = v;
            }
            if (!full) {                                                      // wavefront-uniform
                const int kbase = key0 + lh * 4;
#pragma unroll
                for (int i = 0; i < 32; ++i) {
                    const int key = kbase + (i >> 4) * 32 + ((i >> 2) & 3) * 8 + (i & 3);
                    x[i] = (key >= lo && key < hi) ? x[i] : -INFINITY;
                }
            }
            float mx = x[0];
#pragma unroll
            for (int i = 1; i < 32; ++i) mx = fmaxf(mx, x[i]);
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            // the reference maximum only moves when the tile's maximum exceeds it by more than PF_LAZY:
            // probabilities stay below e^PF_LAZY (exact in the f32 sums, fine in the 16-bit operand) and the
            // 2*D-register rescale of the accumulators becomes rare after the first tiles
            const float m_new = mx > m_run + PF_LAZY ? mx : m_run;
            float alpha = 1.f, rowsum = 0.f;
            if (m_new > -INFINITY) {
                alpha = m_run > -INFINITY ? __builtin_amdgcn_exp2f((m_run - m_new) * LOG2E) : 1.f;
                const float mneg = -m_new * LOG2E;
#pragma unroll
                for (int i = 0; i < 32; ++i) {
                    x[i] = __builtin_amdgcn_exp2f(fmaf(x[i], LOG2E, mneg));      // exp2(-inf) = 0 for masked keys
                    rowsum += x[i];
                }
            } else {
#pragma unroll
                for (int i = 0; i < 32; ++i) x[i] = 0.f;
            }
            rowsum += __shfl_xor(rowsum, 32, 64);
            l_run = l_run * alpha + rowsum;
            m_run = m_new;
            // P^T operand of 16-key step s2: slots 0..7 <- accumulator elements 8*s2 .. 8*s2+7
            u32x4 pf[4];
#pragma unroll
            for (int s2 = 0; s2 < 4; ++s2)
                pf[s2] = u32x4{pack2<KV>(x[8 * s2], x[8 * s2 + 1]), pack2<KV>(x[8 * s2 + 2], x[8 * s2 + 3]),
                               pack2<KV>(x[8 * s2 + 4], x[8 * s2 + 5]), pack2<KV>(x[8 * s2 + 6], x[8 * s2 + 7])};
            // -- O^T += V^T . P^T
            if (__any(alpha != 1.f)) {              // wavefront-uniform and rare after the first tiles
#pragma unroll
                for (int j = 0; j < NJ; ++j)
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc[j][i] *= alpha;
            }
            // key step outermost: consecutive MFMAs go to different accumulators
#pragma unroll
            for (int s2 = 0; s2 < 4; ++s2)
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    const unsigned char *vrow = st + v_off + j * 32 * PF_VROW + s2 * 32;
                    const u32x2 va = *(const u32x2 *)(vrow), vb = *(const u32x2 *)(vrow + 16);
                    acc[j] = mfma32<KV>(u32x4{va.x, va.y, vb.x, vb.y}, pf[s2], acc[j]);
                }
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * PF_AHEAD, 1);
#pragma unroll
            for (int i = 0; i < 4 * NJ - 2 * PF_AHEAD; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 1);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 1);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, 2 * PF_AHEAD, 1);
        }
        if (more) store_v(nx);
        __syncthreads();                                           // also waits for this wavefront's K loads (fence)
    }

    } else {
    // Head sizes 128 and up (64 keeps the serial loop above: its key rows have 8 chunks, too few for the swizzles here).
    // At head size 128 the kernel needs under 256 registers and half the LDS, so two workgroups share a CU and the
    // softmax of one runs beside the MFMAs of the other as well.
    // The loop is software-pipelined over the key tiles: iteration t computes S_t = K_t . Q^T, then the softmax of
    // S_t (vector ALU) TOGETHER WITH O += V_(t-1)^T . P_(t-1) (matrix pipe) - one wavefront per SIMD has nobody else
    // to fill the matrix pipe while it computes exponentials, so it has to overlap the two itself. P_(t-1) and the
    // running statistics of tile t-1 are consistent with the accumulators; the rescale by alpha_t follows the product.
    // LDS: K and V both come by LDS-writing loads, 16-byte chunks in swizzled slots, no register staging. Iteration t
    // requests K_(t+1) into stage (t+1)&1 and V_t into stage t&1 (read by the next iteration's product), one request
    // behind each k-step of S_t; one barrier per tile. The V^T operand of the second product is read with the
    // transposing LDS read (ds_read_b64_tr_b16): within 16 lanes, lane 4r+q supplies the address of 4 consecutive dv
    // of key r and lane i receives keys 0..3 of dv i - the operand layout of the MFMA straight from row-major V.
    // Registers: this file is compiled with MFMA results in vector registers, so the scores feed the softmax without
    // copies and the rare rescale is a plain multiply; the accumulators (D/2), the scores (32) and the operands in
    // flight fill the 256 vector registers, and the Q operand (D/4 registers, read-only) is pinned in accumulation
    // registers, from where the MFMA reads it directly.
    static_assert(CPK >= 16 && Cfg::KROW <= 1024, "chunk swizzles below assume 16..64 chunks per key row");
    static_assert(KK == 2 * NKI, "one tile request per k-step of the first product");
    const int k_swz = l31 & 15;
    const int k_row = l31 * Cfg::KROW;
    // V^T operand addresses: lane = 32*lh + 16*hb + 4*r + q reads key (16*s2 + 8*second + 4*lh + r), dv 32*j + 16*hb + 4*q .. +3.
    // Chunk c of key k sits at slot c ^ 4*(k & 3): the 16 chunks one 32-lane half reads (4 keys x 4 chunks) fall on 16
    // distinct bank groups. (j & 3) meets r in the swizzle, so there is one lane address per j & 3; the rest is immediate.
    // K operand addresses: slot (2*kk + lh) ^ swz = ((kk & 7) ^ (swz >> 1)) * 2 + (lh ^ (swz & 1)) + 16 * (kk >> 3): one lane
    // address per kk & 7, the rest is immediate
    unsigned k_lane[8];
#pragma unroll
    for (int k7 = 0; k7 < 8; ++k7) k_lane[k7] = (unsigned)(k_row + ((((k7 ^ (k_swz >> 1)) << 1) + (lh ^ (k_swz & 1))) << 4));
    const int vhb = (lane >> 4) & 1, vr = (lane >> 2) & 3, vq = lane & 3;
    int v_lane[4];
#pragma unroll
    for (int jj = 0; jj < 4; ++jj)
        v_lane[jj] = Cfg::K_BYTES + (4 * lh + vr) * Cfg::KROW + ((((jj ^ vr) << 2) + 2 * vhb + (vq >> 1)) << 4) + (vq & 1) * 8;

    // cooperative tile loads, 1 KiB (KEYS_PER_KI keys) per instruction. The address is a uniform tile base plus a 32-bit
    // lane offset: a clamp and a 24-bit multiply-add per load. Keys outside the union are read from a clamped in-range key.
    const unsigned row_bytes = (unsigned)kv_row * 2u;
    const int ld_key = lane / CPK, ld_slot = lane % CPK;
    (void)ld_key; (void)ld_slot;                          // used in the device pass only
    struct TileSrc {
        const unsigned char *base;    // uniform
        int rbase, rel_lo, rel_hi;    // uniform: first row of the tile (rolling caches), clamp bounds relative to the tile
    };
    auto tile_src = [&](const unsigned short *src, int t) __attribute__((always_inline)) {
        const int key0 = t * PF_TK;
        TileSrc ts;
        ts.base = (const unsigned char *)(src + kv_base) + (RING ? (size_t)0 : (size_t)key0 * row_bytes);
        ts.rbase = RING ? (int)((unsigned)key0 % (unsigned)ring) : 0;
        ts.rel_lo = g_lo - key0;
        ts.rel_hi = key_clamp_hi - key0;
        return ts;
    };
    auto tile_request = [&](const TileSrc &ts, unsigned char *dst, auto is_v_c, int i) __attribute__((always_inline)) {
#if defined(__HIP_DEVICE_COMPILE__)   // the builtin exists in the device pass only
        constexpr bool IS_V = decltype(is_v_c)::value;
        const int key = (wave * NKI + i) * KEYS_PER_KI + ld_key;
        const int swz = IS_V ? ((key & 3) << 2) : (key & 15);
        int row = ts.rbase + min(max(key, ts.rel_lo), ts.rel_hi);
        if (RING) row = row >= ring ? row - ring : row;
        const unsigned voff = __umul24((unsigned)row, row_bytes) + (unsigned)((ld_slot ^ swz) << 4);
        __builtin_amdgcn_global_load_lds(ts.base + voff, (lds_void *)(dst + (wave * NKI + i) * 1024), 16, 0, 0);
#endif
    };
    using yes = std::integral_constant<bool, true>;
    using no = std::integral_constant<bool, false>;

    f32x16 sc[2];
    u32x4 pf[4] = {};
    const unsigned lds_addr = (unsigned)(size_t)(lds_void *)lds;
    const float qscale = CAP ? 1.f : a.scale;
    const float c2 = qscale * LOG2E;
    auto pin_q = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) asm volatile("" : "+a"(qf[kk]));
    };

    // one tile's front half: S_t = K_t . Q^T with the requests for K of tile t+1 and V of tile t between its MFMAs, then
    // the mask. The LDS reads run PF_AHEAD k-steps ahead of the MFMAs that consume them. Scores stay as the MFMA left
    // them (lane holds keys key0 + kb*32 + (i/4)*8 + lh*4 + i%4 of row l31): the softmax scale rides on the exponent's
    // multiply-add (the launcher sends a scale that is not positive elsewhere), only a soft cap rewrites them.
    auto tile_front = [&](int t) __attribute__((always_inline)) {
        unsigned char *st = lds + ((t - t_begin) & 1) * Cfg::STAGE;
        unsigned char *other = lds + ((t - t_begin + 1) & 1) * Cfg::STAGE;
        // past the end the last K tile is requested once more, into the stage that nobody reads again
        const TileSrc ks = tile_src(kp, min(t + 1, t_end - 1)), vs = tile_src(vp, t);
        // K operands of k-step kk: rows l31 and 32 + l31 at slot (2*kk + lh) ^ swz; written as assembly and waited for
        // by count for the same reason as the V^T operands below
        const unsigned kst = lds_addr + (unsigned)(((t - t_begin) & 1) * Cfg::STAGE);
        auto k_operand = [&](u32x4 (&op)[2], auto kk_c) __attribute__((always_inline)) {
            constexpr int kk = decltype(kk_c)::value;
            const unsigned addr = kst + k_lane[kk & 7];
            asm volatile("ds_read_b128 %0, %2 offset:%3\n\tds_read_b128 %1, %2 offset:%4"
                         : "=&v"(op[0]), "=&v"(op[1]) : "v"(addr), "n"((kk >> 3) * 256), "n"((kk >> 3) * 256 + 32 * Cfg::KROW));
        };
        u32x4 kop[PF_AHEAD][2];
        static_for<0, PF_AHEAD>([&](auto kc) __attribute__((always_inline)) { k_operand(kop[decltype(kc)::value], kc); });
        f32x16 zero;
#pragma unroll
        for (int i = 0; i < 16; ++i) zero[i] = 0.f;
        __builtin_amdgcn_sched_barrier(0);
        static_for<0, KK>([&](auto kc) __attribute__((always_inline)) {
            constexpr int kk = decltype(kc)::value;
            constexpr int later = KK - 1 - kk < PF_AHEAD - 1 ? KK - 1 - kk : PF_AHEAD - 1;   // k-steps requested after this one
            asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(kop[kk % PF_AHEAD][0]), "+v"(kop[kk % PF_AHEAD][1]) : "n"(2 * later));
            sc[0] = mfma32<KV>(kop[kk % PF_AHEAD][0], qf[kk], kk == 0 ? zero : sc[0]);
            sc[1] = mfma32<KV>(kop[kk % PF_AHEAD][1], qf[kk], kk == 0 ? zero : sc[1]);
            if constexpr (kk + PF_AHEAD < KK) k_operand(kop[kk % PF_AHEAD], std::integral_constant<int, kk + PF_AHEAD>{});
            if (kk < NKI) tile_request(ks, other, no{}, kk);
            else tile_request(vs, st + Cfg::K_BYTES, yes{}, kk - NKI);
            __builtin_amdgcn_sched_barrier(0);
        });
        const int key0 = t * PF_TK;
        if (CAP) {
#pragma unroll
            for (int i = 0; i < 32; ++i) sc[i >> 4][i & 15] = a.soft_cap * tanhf(sc[i >> 4][i & 15] * a.scale * cap_inv);
        }
        // No MFMA on the output accumulators inside a branch: the one wavefront-uniform branch of a tile - mask or
        // no mask - sits here, around vector instructions only.
        const bool full = key0 >= w_lo_max && key0 + PF_TK <= w_hi_min;   // every key visible to every row
        if (!full) {
            // key = key0 + 4*lh + c_i is visible iff lo <= key < hi, i.e. (unsigned)(c_i - lo_rel) < span
            const int lo_rel = lo - (key0 + lh * 4);
            const unsigned span = (unsigned)(hi - lo);
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                const int c = (i >> 4) * 32 + ((i >> 2) & 3) * 8 + (i & 3);
                sc[i >> 4][i & 15] = (unsigned)(c - lo_rel) < span ? sc[i >> 4][i & 15] : -INFINITY;
            }
        }
    };
    // The transposing reads are written as assembly: as a builtin the compiler cannot tell them from a read of the
    // stage an LDS-writing load is filling and waits for every load in flight (vmcnt(0)) before the first of them.
    // It does not count them either, so each operand is waited for by count right before its MFMA (v_wait).
    auto v_operand = [&](const unsigned (&vaddr)[4], auto idx_c) __attribute__((always_inline)) {
        constexpr int idx = decltype(idx_c)::value, j = idx % NJ, s2 = idx / NJ;
        constexpr int imm = (j >> 2) * 256 + s2 * 16 * Cfg::KROW;
        u32x2 a0, a1;
        asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4"
                     : "=&v"(a0), "=&v"(a1) : "v"(vaddr[j & 3]), "n"(imm), "n"(imm + 8 * Cfg::KROW));
        return u32x4{a0.x, a0.y, a1.x, a1.y};
    };
    // waits until at most `later` operands requested after this one are still in flight (two reads each)
    auto v_wait = [&](u32x4 &op, auto later_c) __attribute__((always_inline)) {
        asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(op) : "n"(2 * decltype(later_c)::value));
    };
    // the value of the lane 32 away: v_permlane32_swap exchanges the upper half of one register with the lower half of another
    auto other_half_max = [](float x) __attribute__((always_inline)) {
        const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
        return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    };
    auto other_half_sum = [](float x) __attribute__((always_inline)) {
        const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
        return __uint_as_float(r[0]) + __uint_as_float(r[1]);
    };
    // softmax of sc -> pf (next iteration's P^T operand), interleaved with the product of the previous tile
    auto tile_softmax_pv = [&](auto with_pv_c, unsigned vst_off) __attribute__((always_inline)) {
        constexpr bool WITH_PV = decltype(with_pv_c)::value;
        // The softmax is cut into units of a few vector instructions, and the product of the previous tile into its
        // NM MFMAs; the units are dealt out behind the MFMAs by cost (an exponential takes four issue slots) and a
        // scheduling barrier keeps the order (left to itself the compiler issues the whole softmax first and the MFMAs
        // behind it). The V^T operand of MFMA k + PV_AHEAD is requested behind MFMA k.
        //   units 0..7    partial maxima of four scores each (two chains)
        //   unit  8       row maximum across the two lane halves, new reference maximum, alpha, exponent offset
        //   units 9..40   one exponential each, partial sums (two chains)
        //   units 41..44  the four P^T operands of the next product, each written over the operand of this product's
        //                 same key step - so it has to sit behind the last MFMA that reads that one
        //   unit  45      row sum across the lane halves, running sum and maximum
        constexpr int NM = 4 * NJ, PV_AHEAD = NM >= 16 ? 4 : 2;
        static_assert(pf_unit_end(NJ - 1, NM) <= 41 && pf_unit_end(2 * NJ - 1, NM) <= 42 && pf_unit_end(3 * NJ - 1, NM) <= 43 &&
                      pf_unit_end(4 * NJ - 1, NM) <= 44, "a P^T operand would be overwritten before its last MFMA");
        float mxp[2] = {-INFINITY, -INFINITY}, rs[2] = {0.f, 0.f};
        float m_new = m_run, alpha = 1.f, mneg = 0.f;
        auto unit = [&](int u) __attribute__((always_inline)) {
            if (u < 8) {
                // v_max3_f32 by hand: fmaxf on MFMA results first canonicalizes every input (one more instruction per score).
                // The compiler does not see that this assembly reads MFMA results, so the wait states a vector read needs
                // behind the last MFMA that wrote them are put here, once per tile; the other units follow behind these.
                // gfx950: a VALU read of an XDL result needs passes + 4 wait states (12 for the 8-pass 32x32x16 MFMA);
                // PF_SCORE_WAIT adds two of margin. s_nop n gives n + 1 wait states, at most 8 per instruction.
                // This placement relies on the scheduling barriers that keep every MFMA of S_t ahead of unit 0, and the
                // file's build flags (MFMA results in vector registers, kernel arguments preloaded) do not change it.
                if (u == 0) asm volatile("s_nop %0\n\ts_nop %1" ::"n"(7), "n"(PF_SCORE_WAIT - 8 - 1) : "memory");
                float t;
                asm volatile("v_max3_f32 %0, %1, %2, %3" : "=v"(t) : "v"(mxp[u & 1]), "v"(sc[u >> 2][(4 * u) & 15]), "v"(sc[u >> 2][(4 * u + 1) & 15]));
                asm volatile("v_max3_f32 %0, %1, %2, %3" : "=v"(mxp[u & 1]) : "v"(t), "v"(sc[u >> 2][(4 * u + 2) & 15]), "v"(sc[u >> 2][(4 * u + 3) & 15]));
            } else if (u == 8) {
                const float mx = other_half_max(fmaxf(mxp[0], mxp[1])) * qscale;
                // the reference maximum only moves when the tile's maximum exceeds it by more than PF_LAZY:
                // probabilities stay below e^PF_LAZY (exact in the f32 sums, fine in the 16-bit operand) and the
                // D/2-register rescale of the accumulators becomes rare after the first tiles
                m_new = mx > m_run + PF_LAZY ? mx : m_run;
                // branch-free: with nothing visible so far (m_new = -inf) the exponent's offset is 0 and every
                // masked score still gives exp2(-inf) = 0
                alpha = m_run > -INFINITY ? __builtin_amdgcn_exp2f((m_run - m_new) * LOG2E) : 1.f;
                mneg = m_new > -INFINITY ? -m_new * LOG2E : 0.f;
            } else if (u < 41) {
                const int i = u - 9;
                sc[i >> 4][i & 15] = __builtin_amdgcn_exp2f(fmaf(sc[i >> 4][i & 15], c2, mneg));
            } else if (u < 45) {
                const int s2 = u - 41, kb = s2 >> 1, e = (s2 & 1) * 8;
                // P^T operand of 16-key step s2: slots 0..7 <- accumulator elements 8*s2 .. 8*s2+7
                pf[s2] = u32x4{pack2<KV>(sc[kb][e], sc[kb][e + 1]), pack2<KV>(sc[kb][e + 2], sc[kb][e + 3]),
                               pack2<KV>(sc[kb][e + 4], sc[kb][e + 5]), pack2<KV>(sc[kb][e + 6], sc[kb][e + 7])};
                // the row sum takes the probabilities as the product sees them (rounded to the operand type), two per
                // instruction: numerator and denominator of the output then carry the same rounding
                rs[0] = dot2_ones<KV>(pf[s2].x, rs[0]);
                rs[1] = dot2_ones<KV>(pf[s2].y, rs[1]);
                rs[0] = dot2_ones<KV>(pf[s2].z, rs[0]);
                rs[1] = dot2_ones<KV>(pf[s2].w, rs[1]);
            } else if (u == 45) {
                l_run = l_run * alpha + other_half_sum(rs[0] + rs[1]);
                m_run = m_new;
            }
        };
        if (WITH_PV) {
            // -- O^T += V^T . P^T of the previous tile; key step outermost: consecutive MFMAs go to different accumulators
            unsigned vaddr[4];
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) vaddr[jj] = lds_addr + vst_off + (unsigned)v_lane[jj];
            u32x4 vop[PV_AHEAD];
            static_for<0, PV_AHEAD>([&](auto kc) __attribute__((always_inline)) { vop[decltype(kc)::value] = v_operand(vaddr, kc); });
            __builtin_amdgcn_sched_barrier(0);
            static_for<0, NM>([&](auto kc) __attribute__((always_inline)) {
                constexpr int k = decltype(kc)::value;
                v_wait(vop[k % PV_AHEAD], std::integral_constant<int, (NM - 1 - k < PV_AHEAD - 1 ? NM - 1 - k : PV_AHEAD - 1)>{});
                acc[k % NJ] = mfma32<KV>(vop[k % PV_AHEAD], pf[k / NJ], acc[k % NJ]);
                if constexpr (k + PV_AHEAD < NM) vop[k % PV_AHEAD] = v_operand(vaddr, std::integral_constant<int, k + PV_AHEAD>{});
                static_for<pf_unit_end(k, NM), pf_unit_end(k + 1, NM)>([&](auto uc) __attribute__((always_inline)) { unit(decltype(uc)::value); });
                __builtin_amdgcn_sched_barrier(0);
            });
        } else {
#pragma unroll
            for (int u = 0; u < 46; ++u) unit(u);
        }
        if (__any(alpha != 1.f)) {              // wavefront-uniform and rare after the first tiles
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[j][i] *= alpha;
        }
    };

    {
        const TileSrc ks = tile_src(kp, t_begin);
#pragma unroll
        for (int i = 0; i < NKI; ++i) tile_request(ks, lds, no{}, i);
    }
    pin_q();
    __syncthreads();                                               // K of the first tile has landed (fence)
    // first tile, peeled: there is no previous product to overlap with
    tile_front(t_begin);
    tile_softmax_pv(no{}, 0u);
    __syncthreads();
    for (int t = t_begin + 1; t < t_end; ++t) {
        pin_q();
        tile_front(t);
        tile_softmax_pv(yes{}, (unsigned)(((t - t_begin + 1) & 1) * Cfg::STAGE));
        __syncthreads();                                           // also waits for this wavefront's tile requests (fence)
    }
    {   // the last tile's product
        constexpr int NM = 4 * NJ, PV_AHEAD = 4;
        unsigned vaddr[4];
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) vaddr[jj] = lds_addr + (unsigned)(((t_end - 1 - t_begin) & 1) * Cfg::STAGE) + (unsigned)v_lane[jj];
        u32x4 vop[PV_AHEAD];
        static_for<0, PV_AHEAD>([&](auto kc) __attribute__((always_inline)) { vop[decltype(kc)::value] = v_operand(vaddr, kc); });
        __builtin_amdgcn_sched_barrier(0);
        static_for<0, NM>([&](auto kc) __attribute__((always_inline)) {
            constexpr int k = decltype(kc)::value;
            v_wait(vop[k % PV_AHEAD], std::integral_constant<int, (NM - 1 - k < PV_AHEAD - 1 ? NM - 1 - k : PV_AHEAD - 1)>{});
            acc[k % NJ] = mfma32<KV>(vop[k % PV_AHEAD], pf[k / NJ], acc[k % NJ]);
            if constexpr (k + PV_AHEAD < NM) vop[k % PV_AHEAD] = v_operand(vaddr, std::integral_constant<int, k + PV_AHEAD>{});
            __builtin_amdgcn_sched_barrier(0);
        });
    }
    }

    if (HP && nseg > 1) {
        // f16 accumulators under a per-row power of two: 2^e <= max|acc| < 2^(e+1) (e clamped so that its inverse is a
        // normal number; a row of zeros takes 1)
        float amax = 0.f;
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(acc[j][i]));
        amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
        unsigned e = (__float_as_uint(amax) >> 23) & 0xFFu;
        e = e == 0u ? 127u : min(e, 253u);
        const float down = __uint_as_float((254u - e) << 23);
        if (row_ok) {
            if (lh == 0) {
                part_stats[r & 15] = m_run;
                part_stats[16 + (r & 15)] = l_run;
                part_stats[32 + (r & 15)] = __uint_as_float(e << 23);
            }
            unsigned char *o = part + (r & 15) * (D * 2) + lh * 32;
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                unsigned w[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) w[i] = pack2<AIONHIP_F16>(acc[j][2 * i] * down, acc[j][2 * i + 1] * down);
                *(u32x4 *)(o + j * 64) = u32x4{w[0], w[1], w[2], w[3]};
                *(u32x4 *)(o + j * 64 + 16) = u32x4{w[4], w[5], w[6], w[7]};
            }
        }
    } else if (row_ok) {
        const float inv = nseg > 1 ? 1.f : (l_run > 0.f ? 1.f / l_run : 0.f);          // empty interval -> zeros
        float *o = nseg > 1 ? (float *)part + (r & 15) * D : a.out + qbase;
        if (nseg > 1 && lh == 0) {
            part_stats[r & 15] = m_run;
            part_stats[16 + (r & 15)] = l_run;
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const f32x4 v = f32x4{acc[j][q4 * 4], acc[j][q4 * 4 + 1], acc[j][q4 * 4 + 2], acc[j][q4 * 4 + 3]} * inv;
                *(f32x4 *)(o + j * 32 + q4 * 8 + lh * 4) = v;
            }
    }
}

// The same merge for many rows and few segments (the prefill kernel's key segments): one thread per (row, four
// consecutive dv), so that a wavefront reads whole contiguous rows of every segment's accumulators.
__device__ __forceinline__ float half_bits_to_float(unsigned bits) { return (float)__builtin_bit_cast(_Float16, (unsigned short)bits); }

template <int D, bool HP>
__global__ __launch_bounds__(256) void attn_merge_rows_kernel(AttnArgs a) {
    constexpr int PART_BYTES = pf_partial_bytes(D, HP);
    constexpr int TPR = D / 4, RPB = 256 / TPR;          // threads per row, rows per workgroup
    constexpr int UN = 4;
    const int unit = blockIdx.y, b = unit / a.Hkv, hk = unit % a.Hkv;
    const int rr = blockIdx.x * RPB + (int)threadIdx.x / TPR, dv = ((int)threadIdx.x % TPR) * 4;
    if (rr >= a.rows_total) return;
    const int rt = rr >> 4, row = rr & 15;
    const unsigned char *base = (const unsigned char *)a.partial + (size_t)(unit * a.row_tiles + rt) * a.nseg * PART_BYTES;
    // f16 form: where dv .. dv+3 stand in the row (the order the tile kernel's lanes hold them)
    const int pos = (dv & ~31) + ((dv >> 2) & 1) * 16 + ((dv >> 3) & 3) * 4;
    float m_all = -INFINITY, l_all = 0.f;
    f32x4 o = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < a.nseg; s0 += UN) {
        float ms[UN], ls[UN];
        f32x4 os[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const unsigned char *p = base + (size_t)min(s0 + u, a.nseg - 1) * PART_BYTES;      // clamped: every load is unconditional
            const float *st = (const float *)(p + (HP ? 32 * D : 64 * D));
            ms[u] = st[row];
            ls[u] = st[16 + row];
            if (HP) {
                const u32x2 h = *(const u32x2 *)(p + (row * D + pos) * 2);
                const float sc = st[32 + row];
                const unsigned w0 = h.x, w1 = h.y;
                os[u] = f32x4{half_bits_to_float(w0 & 0xFFFFu), half_bits_to_float(w0 >> 16), half_bits_to_float(w1 & 0xFFFFu),
                              half_bits_to_float(w1 >> 16)} * sc;
            } else {
                os[u] = *(const f32x4 *)((const float *)p + row * D + dv);
            }
        }
        float m_new = m_all;
#pragma unroll
        for (int u = 0; u < UN; ++u)
            if (s0 + u < a.nseg) m_new = fmaxf(m_new, ms[u]);
        if (m_new > -INFINITY) {
            const float f0 = m_all > -INFINITY ? exp2f((m_all - m_new) * LOG2E) : 0.f;
            o *= f0;
            l_all *= f0;
#pragma unroll
            for (int u = 0; u < UN; ++u) {
                const bool live = s0 + u < a.nseg && ms[u] > -INFINITY;
                const float f = live ? exp2f((ms[u] - m_new) * LOG2E) : 0.f;
                o += os[u] * f;
                l_all += ls[u] * f;
            }
            m_all = m_new;
        }
    }
    const int l2 = rr / a.groups, g3 = rr % a.groups;
    const float inv = l_all > 0.f ? 1.f / l_all : 0.f;
    *(f32x4 *)(a.out + (((size_t)b * a.L + l2) * a.Hq + hk * a.groups + g3) * D + dv) = o * inv;
}

template <int KV, int D, bool RING>
int launch_prefill_t(aionhip_ctx *ctx, AttnArgs &a) {
    using PCfg = PrefillCfg<D>;
    const int units = a.B * a.Hkv;
    const int cus0 = ctx->cu_count > 0 ? ctx->cu_count : 256;
    // No more workgroups than CUs: the key range of every row tile is cut into segments (at least
    // PF_SEG_TILES tiles each) and the partial results are merged, as in the decode path. Measured at 8 heads
    // x head size 256: L = 4096 (256 workgroups) 167 -> 136 us with two segments, L = 3072 125 -> 90 us.
    const int wgs = units * ((a.rows_total + PF_ROWS - 1) / PF_ROWS);
    const int key_tiles = (a.T + PF_TK - 1) / PF_TK;
    // A tile of head size 128 or less is half the work and two workgroups share a CU: a segment is worth eight tiles there, and
    // two segments for balance only pay from 32 key tiles on (8 kv heads x 4 query heads each, L = 1024: 26 us in one
    // segment, 35 in two; one kv head x 8, L = 2048: 40 against 33).
    const int seg_tiles = D > 128 ? PF_SEG_TILES : 2 * PF_SEG_TILES;
    const bool balance_pays = key_tiles >= (D > 128 ? 40 : 32);     // (head size 256, 2 kv heads x 8, L = 2048, 32 key tiles: 63 us in one segment, 78 in two)
    int want = cus0 / max(wgs, 1);
    if (want < 2 && wgs <= cus0 && balance_pays) want = 2;      // one round of workgroups: two segments even out what a causal mask skews
    // Between one and two rounds the longest row tile alone takes as long as two average ones (under a causal mask a tile's
    // work grows with its index): the device is busy wgs / (2 * CUs) of the time. Two segments halve the longest piece;
    // they pay while that gain exceeds the merge pass (measured at 8 heads x head size 256: 260 workgroups 109 -> 94 us, 288
    // 122 -> 116, 320 the same, 352 and more slower).
    if (want < 2 && D > 128 && wgs > cus0 && balance_pays && (long)wgs * 10 < (long)cus0 * PF_TWO_SEG_BELOW_TENTHS) want = 2;
    int nseg = max(1, min(min(want, key_tiles / seg_tiles), 16));
    a.nseg = nseg;
    if (nseg > 1) {
        const size_t bytes = (size_t)units * a.row_tiles * nseg * pf_partial_bytes(D, pf_half_partials(KV));
        int rc = ensure_scratch2(ctx, bytes);
        if (rc) return rc;
        a.partial = (float *)ctx->scratch2;
    }
    static bool attr_pf[2] = {false, false};   // per kernel instantiation
    const bool cap = a.soft_cap > 0.f;
    const void *fn = cap ? (const void *)attn_prefill_kernel<KV, D, true, RING> : (const void *)attn_prefill_kernel<KV, D, false, RING>;
    if (!attr_pf[cap]) {
        HIP_TRY(ctx, hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, PCfg::LDS_BYTES));
        attr_pf[cap] = true;
    }
    {
        ProfScope scope(ctx, "attn_prefill");
        const dim3 grid((unsigned)((a.rows_total + PF_ROWS - 1) / PF_ROWS), (unsigned)units, (unsigned)nseg);
        if (cap) launch_k(ctx, attn_prefill_kernel<KV, D, true, RING>, grid, dim3(256), PCfg::LDS_BYTES, a);
        else launch_k(ctx, attn_prefill_kernel<KV, D, false, RING>, grid, dim3(256), PCfg::LDS_BYTES, a);
    }
    if (nseg > 1) {
        ProfScope scope(ctx, "attn_merge");
        constexpr int RPB = 256 / (D / 4);
        launch_k(ctx, attn_merge_rows_kernel<D, pf_half_partials(KV)>, dim3((unsigned)((a.rows_total + RPB - 1) / RPB), (unsigned)units), dim3(256), 0, a);
    }
    LAUNCH_CHECK(ctx, "attn_prefill");
    return AIONHIP_OK;
}

template <int KV>
int launch_prefill_d(aionhip_ctx *ctx, AttnArgs &a, int d) {
    if (a.ring) {
        if (d == 64) return launch_prefill_t<KV, 64, true>(ctx, a);
        if (d == 128) return launch_prefill_t<KV, 128, true>(ctx, a);
        return launch_prefill_t<KV, 256, true>(ctx, a);
    }
    if (d == 64) return launch_prefill_t<KV, 64, false>(ctx, a);
    if (d == 128) return launch_prefill_t<KV, 128, false>(ctx, a);
    return launch_prefill_t<KV, 256, false>(ctx, a);
}

}  // namespace

namespace attn {

bool prefill_takes(const AttnArgs &a, int d) {
    if (d != 64 && d != 128 && d != 256) return false;
    if (a.kv_dtype != AIONHIP_F16 && a.kv_dtype != AIONHIP_BF16) return false;
    if (d >= PF_PIPE_D) {
        // the pipelined loop folds the softmax scale into the exponent (it takes the row maximum of the unscaled
        // scores) and addresses the rows of a rolling cache by 32-bit byte offsets
        if (!(a.scale > 0.f)) return false;
        if (a.ring && (size_t)a.T * a.Hkv * d * 2 >= ((size_t)1 << 32)) return false;
    }
    return true;
}

int launch_prefill(aionhip_ctx *ctx, AttnArgs &a, int d) {
    if (a.kv_dtype == AIONHIP_F16) return launch_prefill_d<AIONHIP_F16>(ctx, a, d);
    return launch_prefill_d<AIONHIP_BF16>(ctx, a, d);
}

}  // namespace attn
