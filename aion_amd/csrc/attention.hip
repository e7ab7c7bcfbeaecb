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
// attn_prefill_kernel - many query rows: 128 rows per workgroup, K/V tiles shared through LDS, 32x32x16 MFMA
//   (described at the kernel).
// attn_generic_kernel - any head size / f32 K,V: one wavefront per query row, scores staged in
//   global scratch. Slow; it exists so that every shape the op allows has a GPU path.
//
// Softmax uses exp2 on (s - m) * log2(e); aion's CPU path uses a 4th-order polynomial exp
// (cpu/kernels/fast_math.zig:79-92, rel. err 4e-5), so results agree to ~1e-4, not bitwise.
#include "common.h"

#include <climits>
#include <type_traits>

namespace {

using f16x8 = __attribute__((ext_vector_type(8))) _Float16;
using bf16x8 = __attribute__((ext_vector_type(8))) __bf16;

constexpr float LOG2E = 1.4426950408889634f;
constexpr int TILE_KEYS = 32;

struct AttnArgs {
    const void *q, *k, *v;
    float *out;
    const int *positions, *kv_lengths;
    float *partial;
    int B, L, T, Hq, Hkv, groups, rows_total, row_tiles, nseg;
    int ring;      // rolling caches: T (logical key t lives in row t % T); 0: row t is key t
    int q_dtype, kv_dtype;
    float scale, soft_cap;
    unsigned win_left, win_right, win_chunk;
};

__device__ __forceinline__ unsigned short f32_to_bf16_bits(float x) {
    unsigned u = __float_as_uint(x);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
}
__device__ __forceinline__ float bf16_bits_to_f32(unsigned short b) { return __uint_as_float((unsigned)b << 16); }

template <int KV>
__device__ __forceinline__ unsigned short to_half_bits(float x) {
    if (KV == AIONHIP_F16) return __half_as_ushort(__float2half_rn(x));
    return f32_to_bf16_bits(x);
}
template <int KV>
__device__ __forceinline__ float from_half_bits(unsigned short b) {
    if (KV == AIONHIP_F16) return __half2float(__ushort_as_half(b));
    return bf16_bits_to_f32(b);
}
// two f32 -> one 32-bit word of two halves (RNE), low half first
using f32x2 = __attribute__((ext_vector_type(2))) float;
using bf16x2 = __attribute__((ext_vector_type(2))) __bf16;
template <int KV>
__device__ __forceinline__ unsigned pack2(float a, float b) {
    if (KV == AIONHIP_F16) {
        const __half2 h = __floats2half2_rn(a, b);
        return *reinterpret_cast<const unsigned *>(&h);
    }
    // one v_cvt_pk_bf16_f32 (round to nearest even) instead of integer rounding per element
    return __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2{a, b}, bf16x2));
}
template <int KV>
__device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
    if (KV == AIONHIP_F16)
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

__device__ __forceinline__ float load_scalar(const void *p, int dtype, size_t i) {
    if (dtype == AIONHIP_F32) return ((const float *)p)[i];
    if (dtype == AIONHIP_F16) return __half2float(((const __half *)p)[i]);
    return bf16_bits_to_f32(((const unsigned short *)p)[i]);
}

// AttentionWindow.keys (aion graph/graph.zig:160-167)
__device__ __forceinline__ void window_keys(unsigned left, unsigned right, unsigned chunk, int pos, int kv_end, int &lo, int &hi) {
    const long anchor = chunk > 0 ? (long)(pos / (int)chunk) * (int)chunk : pos;
    const long span = chunk > 0 ? chunk : 1;
    const long l = anchor - (anchor < (long)left ? anchor : (long)left);
    long h = right == 0xFFFFFFFFu ? (long)INT_MAX : anchor + span + (long)right;
    if (h > kv_end) h = kv_end;
    lo = (int)l;
    hi = (int)h;
}

// Rolling caches (aion storage/cache.zig:202-207, cpu/exec/attention.zig:1072-1075, 1150-1152): the cache length may
// exceed the capacity, keys older than length - capacity are gone, and key t is read from row t % capacity.
__device__ __forceinline__ int phys_key(int ring, int t) { return ring ? (int)((unsigned)t % (unsigned)ring) : t; }
// The same for the keys of one tile, whose first key key0 is uniform: one modulo per tile (base), then an add and
// a conditional subtract per key. Valid while a tile is no longer than the ring (the launcher sees to that).
struct TileMap {
    int key0, base, wrap;
    __device__ __forceinline__ TileMap(int ring, int k0) : key0(k0), base(ring ? (int)((unsigned)k0 % (unsigned)ring) : k0), wrap(ring ? ring : INT_MAX) {}
    __device__ __forceinline__ int row(int key) const {
        const int r = base + (key - key0);
        return r >= wrap ? r - wrap : r;
    }
};
__device__ __forceinline__ int clip_kv_end(int ring, int t_cap, int kv_end_raw) {
    return ring ? max(0, kv_end_raw) : max(0, min(kv_end_raw, t_cap));
}
__device__ __forceinline__ void clip_to_ring(int ring, int kv_end, int &lo, int &hi) {
    if (ring) lo = max(lo, kv_end - ring);
    if (hi < lo) hi = lo;
}

__device__ __forceinline__ int wave_min_i(int v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = min(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ int wave_max_i(int v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = max(v, __shfl_xor(v, o, 64));
    return v;
}

// NW = wavefronts per workgroup: 4 in prefill mode, 8 in split mode (a decode over a short cache
// is one workgroup whose eight wavefronts take one 32-key tile each)
template <int D, int NW>
struct FlashCfg {
    static constexpr int ROW_BYTES = D * 2;                      // unpadded: the tile is filled by LDS-writing loads
    static constexpr int WAVE_LDS = TILE_KEYS * ROW_BYTES;       // one V tile per wavefront
    static constexpr int WG_LDS = NW * WAVE_LDS;
    static constexpr int MERGE_LDS = (NW * (16 * (D + 4) + 32) + 16 * NW + 32) * 4;   // split mode: NW x (acc[16][D+4], m[16], l[16]) f32 + merge factors
    static constexpr int Q_ROW = D * 2 + 64;                     // split mode: the 16 query rows in the K/V element type
    static constexpr int Q_OFF = WG_LDS > MERGE_LDS ? WG_LDS : MERGE_LDS;
    static constexpr int LDS_BYTES = Q_OFF + 16 * Q_ROW;
};
constexpr int SPLIT_NW = 8;

// HILO: q and the probabilities are fed to the MFMAs as a high and a low half-precision part
// (x = hi + lo, ~2x the mantissa), which keeps an f32 query path at f32-level accuracy; used when
// q arrives as f32 (aion's cached decode: f32 q over an f16 cache). K and V are exact either way.
// RING: the caches are rolling rings (a.ring = T). A template flag, not a run-time test: the identity instances
// must not carry the ring's extra live values (both kernels sit at their register limit).
template <int KV, int D, bool SPLIT, bool HILO, bool RING = false>
__global__ __launch_bounds__(SPLIT ? SPLIT_NW * 64 : 256) void attn_flash_kernel(AttnArgs a) {
    const int ring = RING ? a.ring : 0;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    constexpr int NW = SPLIT ? SPLIT_NW : 4;
    using Cfg = FlashCfg<D, NW>;
    constexpr int KK = D / 32;   // MFMA k-steps over the head dim
    constexpr int MT = D / 16;   // 16-wide dv tiles

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = lane & 15, g = lane >> 4;
    const int unit = blockIdx.y;
    const int b = unit / a.Hkv, hk = unit % a.Hkv;
    int rt, seg;
    if (SPLIT) { rt = blockIdx.x / a.nseg; seg = blockIdx.x % a.nseg; }
    else { rt = blockIdx.x * 4 + wave; seg = 0; }

    // ---- this lane's query row. Loads are requested in dependency order and consumed late: the index
    // operands first, then q (its address needs no loaded value), so one memory round trip covers both.
    const int r = rt * 16 + n;
    const bool row_ok = rt < a.row_tiles && r < a.rows_total;
    const int li = row_ok ? r / a.groups : 0, gi = row_ok ? r % a.groups : 0;
    const int hq = hk * a.groups + gi;
    // The cache length is read with a vector load (a per-lane zero in the address keeps the compiler from
    // turning it into a scalar load, which it would wait for on the spot): it is then in flight together with
    // the position and the query loads instead of ahead of them.
    // Both loads are unconditional (an absent operand reads a word of q instead and is replaced afterwards): a
    // load under a branch is waited for at the end of its block.
    const int lane_zero = (int)__builtin_amdgcn_mbcnt_lo(0u, 0u);
    const int *len_p = a.kv_lengths ? a.kv_lengths + b : (const int *)a.q;
    const int *pos_p = a.positions ? a.positions + ((size_t)b * a.L + li) : (const int *)a.q;
    const int len_ld = len_p[lane_zero], pos_ld = *pos_p;
    const int kv_end_raw = a.kv_lengths ? len_ld : a.T;
    const int pos_raw = (row_ok && a.positions) ? pos_ld : li;

    const size_t qbase = (((size_t)b * a.L + li) * a.Hq + hq) * D;
    const bool q_f32_vec = a.q_dtype == AIONHIP_F32 && (((uintptr_t)a.q) & 15) == 0;
    const bool q_same = a.q_dtype == KV && (((uintptr_t)a.q) & 15) == 0;
    u32x4 qf[KK], qf_lo[HILO ? KK : 1];
    f32x4 qx0[KK], qx1[KK];
    // split mode, f32 queries: every wavefront needs the same 16 rows, so the workgroup fetches them once
    // (two 16-byte loads per thread instead of 2*KK per lane of every wavefront through the one L1), converts
    // and shares them through LDS; the fragments are read back after the first tile's K/V loads are issued.
    const bool q_shared = SPLIT && !HILO && q_f32_vec && D * 16 / 8 <= NW * 64;
    f32x4 qs0 = f32x4{0.f, 0.f, 0.f, 0.f}, qs1 = qs0;
    constexpr int QT = D / 8;                                    // threads per staged row (8 elements each)
    const int qs_row = threadIdx.x / QT, qs_col = (threadIdx.x % QT) * 8;
    if (q_shared) {
        const int r2 = rt * 16 + qs_row;
        if (qs_row < 16 && rt < a.row_tiles && r2 < a.rows_total) {
            const int l2 = r2 / a.groups, g2 = r2 % a.groups;
            const f32x4 *qp = (const f32x4 *)((const float *)a.q + (((size_t)b * a.L + l2) * a.Hq + hk * a.groups + g2) * D + qs_col);
            qs0 = qp[0];
            qs1 = qp[1];
        }
    } else
    if (q_same) {                    // already in the MFMA element type: one 16-byte load per k-step
#pragma unroll
        for (int kk = 0; kk < KK; ++kk)
            qf[kk] = *(const u32x4 *)((const unsigned short *)a.q + qbase + kk * 32 + g * 8);
    } else if (q_f32_vec) {
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const f32x4 *qp = (const f32x4 *)((const float *)a.q + qbase + kk * 32 + g * 8);
            qx0[kk] = qp[0];
            qx1[kk] = qp[1];
        }
    }

    int kv_end = clip_kv_end(ring, a.T, kv_end_raw);
    int lo = 0, hi = 0;
    if (row_ok) {
        window_keys(a.win_left, a.win_right, a.win_chunk, max(pos_raw, 0), kv_end, lo, hi);
        clip_to_ring(ring, kv_end, lo, hi);
    }
    const int uni_lo = wave_min_i(hi > lo ? lo : INT_MAX);
    const int uni_hi = wave_max_i(hi > lo ? hi : 0);

    // ---- Q^T operand: 8 consecutive d of row n per k-step, converted to the K/V element type
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
        if (q_shared) break;
        if (q_same) {
            if (!row_ok) qf[kk] = u32x4{0u, 0u, 0u, 0u};
            if (HILO) qf_lo[kk] = u32x4{0u, 0u, 0u, 0u};
            continue;
        }
        float x[8];
        if (q_f32_vec) {
            x[0] = qx0[kk].x; x[1] = qx0[kk].y; x[2] = qx0[kk].z; x[3] = qx0[kk].w;
            x[4] = qx1[kk].x; x[5] = qx1[kk].y; x[6] = qx1[kk].z; x[7] = qx1[kk].w;
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) x[j] = load_scalar(a.q, a.q_dtype, qbase + kk * 32 + g * 8 + j);
        }
        if (!HILO) {
#pragma unroll
            for (int j = 0; j < 8; ++j) x[j] = row_ok ? x[j] : 0.f;
            qf[kk] = u32x4{pack2<KV>(x[0], x[1]), pack2<KV>(x[2], x[3]), pack2<KV>(x[4], x[5]), pack2<KV>(x[6], x[7])};
            continue;
        }
        unsigned short h[8], lo8[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float xv = row_ok ? x[j] : 0.f;
            h[j] = to_half_bits<KV>(xv);
            lo8[j] = HILO ? to_half_bits<KV>(xv - from_half_bits<KV>(h[j])) : (unsigned short)0;
        }
        qf[kk] = u32x4{(unsigned)h[0] | ((unsigned)h[1] << 16), (unsigned)h[2] | ((unsigned)h[3] << 16),
                       (unsigned)h[4] | ((unsigned)h[5] << 16), (unsigned)h[6] | ((unsigned)h[7] << 16)};
        if (HILO)
            qf_lo[kk] = u32x4{(unsigned)lo8[0] | ((unsigned)lo8[1] << 16), (unsigned)lo8[2] | ((unsigned)lo8[3] << 16),
                              (unsigned)lo8[4] | ((unsigned)lo8[5] << 16), (unsigned)lo8[6] | ((unsigned)lo8[7] << 16)};
    }

    f32x4 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;

    // ---- key tiles of this wavefront
    int t_begin = 0, t_end = 0, t_step = 1;
    if (uni_hi > uni_lo) {
        const int tb = uni_lo / TILE_KEYS, te = (uni_hi + TILE_KEYS - 1) / TILE_KEYS;
        if (SPLIT) {
            const int per = (te - tb + a.nseg - 1) / a.nseg;
            t_begin = tb + seg * per + wave;
            t_end = min(tb + (seg + 1) * per, te);
            t_step = NW;
        } else {
            t_begin = tb;
            t_end = te;
        }
    }

    unsigned char *vs = lds + wave * Cfg::WAVE_LDS;
    const unsigned short *kp = (const unsigned short *)a.k;
    const unsigned short *vp = (const unsigned short *)a.v;
    const size_t kv_row = (size_t)a.Hkv * D;                     // elements between consecutive tokens
    const size_t kv_base = ((size_t)b * a.T * a.Hkv + hk) * D;

    // K (MFMA operand layout, registers) of a tile is requested one tile ahead, right after the S MFMAs
    // have released the registers. V goes global -> LDS directly (global_load_lds_dwordx4, 1 KiB per
    // instruction) into this wavefront's tile, requested as soon as the previous tile's gathers are done.
    // Tile layout: key row of D*2 bytes, 16-byte chunk c of key k at slot c ^ (2 * ((k >> 2) & 3)): the
    // four key groups of a gather then read distinct banks. Keys outside the union interval are read from
    // a clamped in-range key instead (their probabilities are exact zeros, and the cache tail may hold
    // anything, so the value must only be finite).
    constexpr int NVI = TILE_KEYS * D * 2 / 1024;
    constexpr int KEYS_PER_VI = 1024 / (D * 2);
    // Addresses: while one batch entry's cache is under 2 GiB (a uniform test) a row is reached by a 32-bit byte
    // offset from a uniform base - one 24-bit multiply-add per load instead of 64-bit arithmetic, which counts
    // when a lone workgroup issues a whole short cache's loads.
    const unsigned row_bytes = (unsigned)(kv_row * 2);
    const bool near = (size_t)a.T * kv_row * 2 < ((size_t)1 << 31) && a.T < (1 << 24) && row_bytes < (1u << 24);
    const unsigned char *kb8 = (const unsigned char *)(kp + kv_base), *vb8 = (const unsigned char *)(vp + kv_base);
    const int k_last = RING ? max(uni_hi - 1, 0) : a.T - 1;        // the last key a K load may name
    u32x4 kf[2][KK];
    auto load_k_as = [&](int t, auto near_c) __attribute__((always_inline)) {
        constexpr bool near = decltype(near_c)::value;
        const int key0 = t * TILE_KEYS;
        const TileMap tm(ring, key0);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int kabs = tm.row(min(key0 + h * 16 + n, k_last));
            if (near) {
                const unsigned char *krow = kb8 + (__umul24((unsigned)kabs, row_bytes) + (unsigned)g * 16u);
#pragma unroll
                for (int kk = 0; kk < KK; ++kk) kf[h][kk] = *(const u32x4 *)(krow + kk * 64);
            } else {
                const unsigned short *krow = kp + kv_base + (size_t)kabs * kv_row + g * 8;
#pragma unroll
                for (int kk = 0; kk < KK; ++kk) kf[h][kk] = *(const u32x4 *)(krow + kk * 32);
            }
        }
    };
    const int v_key_in = (lane * 16) / (D * 2);                      // key of this lane within one V load
    const int v_slot = ((lane * 16) % (D * 2)) / 16;                 // its 16-byte slot within the key row
    const int v_hi_key = max(uni_hi - 1, 0);
    auto load_k = [&](int t) __attribute__((always_inline)) {
        if (near) load_k_as(t, std::true_type{});
        else load_k_as(t, std::false_type{});
    };
    auto load_v_as = [&](int t, auto near_c) __attribute__((always_inline)) {
#if defined(__HIP_DEVICE_COMPILE__)   // the builtin exists in the device pass only
        constexpr bool near = decltype(near_c)::value;
        const int key0 = t * TILE_KEYS;
        const TileMap tm(ring, key0);
#pragma unroll
        for (int i = 0; i < NVI; ++i) {
            const int key = i * KEYS_PER_VI + v_key_in;
            // (key >> 2) & 3 does not depend on the lane while an instruction covers at most four keys
            const int grp = KEYS_PER_VI <= 4 ? ((i * KEYS_PER_VI) >> 2) & 3 : (key >> 2) & 3;
            const int chunk = v_slot ^ (2 * grp);
            const int kabs = tm.row(min(max(key0 + key, uni_lo), v_hi_key));
            if (near)
                __builtin_amdgcn_global_load_lds(vb8 + (__umul24((unsigned)kabs, row_bytes) + (unsigned)chunk * 16u), (lds_void *)(vs + i * 1024), 16, 0, 0);
            else
                __builtin_amdgcn_global_load_lds(vp + kv_base + (size_t)kabs * kv_row + chunk * 8, (lds_void *)(vs + i * 1024), 16, 0, 0);
        }
#endif
    };
    auto load_v = [&](int t) __attribute__((always_inline)) {
        if (near) load_v_as(t, std::true_type{});
        else load_v_as(t, std::false_type{});
    };
    if (t_begin < t_end) {
        load_k(t_begin);
        load_v(t_begin);
    }
    if (q_shared) {
        unsigned char *qsm = lds + Cfg::Q_OFF;
        if (qs_row < 16)
            *(u32x4 *)(qsm + qs_row * Cfg::Q_ROW + qs_col * 2) =
                u32x4{pack2<KV>(qs0.x, qs0.y), pack2<KV>(qs0.z, qs0.w), pack2<KV>(qs1.x, qs1.y), pack2<KV>(qs1.z, qs1.w)};
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) qf[kk] = *(const u32x4 *)(qsm + n * Cfg::Q_ROW + kk * 64 + g * 16);
    }
    for (int t = t_begin; t < t_end; t += t_step) {
        const int key0 = t * TILE_KEYS;
        const bool more = t + t_step < t_end;      // wavefront-uniform
        // -- S^T = K . Q^T for two 16-key halves
        f32x4 s[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            f32x4 c = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                c = mfma16<KV>(kf[h][kk], qf[kk], c);
                if (HILO) c = mfma16<KV>(kf[h][kk], qf_lo[kk], c);
            }
            s[h] = c;
        }
        if (more) load_k(t + t_step);
        // -- scale, soft cap, interval mask; lane holds keys key0 + h*16 + g*4 + i of row n
        float p[8];
        float mx = -INFINITY;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = key0 + h * 16 + g * 4 + i;
                float x = s[h][i] * a.scale;
                if (a.soft_cap > 0.f) x = a.soft_cap * tanhf(x / a.soft_cap);
                const bool ok = key >= lo && key < hi;
                x = ok ? x : -INFINITY;
                p[h * 4 + i] = x;
                mx = fmaxf(mx, x);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        float alpha = 1.f, rowsum = 0.f;
        if (m_new > -INFINITY) {
            alpha = m_run > -INFINITY ? exp2f((m_run - m_new) * LOG2E) : 1.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                p[j] = p[j] > -INFINITY ? exp2f((p[j] - m_new) * LOG2E) : 0.f;
                rowsum += p[j];
            }
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) p[j] = 0.f;
        }
        rowsum += __shfl_xor(rowsum, 16, 64);
        rowsum += __shfl_xor(rowsum, 32, 64);
        l_run = l_run * alpha + rowsum;
        m_run = m_new;
        unsigned short ph[8], pl[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            ph[j] = to_half_bits<KV>(p[j]);
            pl[j] = HILO ? to_half_bits<KV>(p[j] - from_half_bits<KV>(ph[j])) : (unsigned short)0;
        }
        const u32x4 pf = u32x4{(unsigned)ph[0] | ((unsigned)ph[1] << 16), (unsigned)ph[2] | ((unsigned)ph[3] << 16),
                               (unsigned)ph[4] | ((unsigned)ph[5] << 16), (unsigned)ph[6] | ((unsigned)ph[7] << 16)};
        const u32x4 pf_lo = u32x4{(unsigned)pl[0] | ((unsigned)pl[1] << 16), (unsigned)pl[2] | ((unsigned)pl[3] << 16),
                                  (unsigned)pl[4] | ((unsigned)pl[5] << 16), (unsigned)pl[6] | ((unsigned)pl[7] << 16)};

        // -- this tile's V has landed in the wavefront's LDS tile once only the younger K loads are
        //    outstanding (loads complete in order); the tile is written and read by this wavefront only
        if (more) __builtin_amdgcn_s_waitcnt(vmcnt_imm(2 * KK));
        else __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));

        // -- O^T += V^T . P^T ; operand slot j of lane group g is key g*4+j (j<4) / 16+g*4+j-4
        const bool rescale = __any(alpha != 1.f);     // wavefront-uniform: skip 4*MT multiplies when no row's max moved
        // element (key, dv) sits at key*ROW + ((dv/8) ^ 2g)*16 + (dv%8)*2; (key >> 2) & 3 == g for all 8 keys of a lane
        const unsigned char *vcol = vs + (n & 7) * 2;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            unsigned short e[8];
            const int coff = ((mt * 2 + (n >> 3)) ^ (2 * g)) * 16;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int key = j < 4 ? g * 4 + j : 16 + g * 4 + (j - 4);
                e[j] = *(const unsigned short *)(vcol + key * Cfg::ROW_BYTES + coff);
            }
            const u32x4 vf = u32x4{(unsigned)e[0] | ((unsigned)e[1] << 16), (unsigned)e[2] | ((unsigned)e[3] << 16),
                                   (unsigned)e[4] | ((unsigned)e[5] << 16), (unsigned)e[6] | ((unsigned)e[7] << 16)};
            f32x4 c = acc[mt];
            if (rescale) c *= alpha;
            c = mfma16<KV>(vf, pf, c);
            if (HILO) c = mfma16<KV>(vf, pf_lo, c);
            acc[mt] = c;
        }
        if (more) load_v(t + t_step);      // the gathers above are complete: their values fed the MFMAs
    }

    if (!SPLIT) {
        if (row_ok) {
            const float inv = l_run > 0.f ? 1.f / l_run : 0.f;      // empty interval -> zeros
            float *o = a.out + (((size_t)b * a.L + li) * a.Hq + hq) * D + g * 4;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) *(f32x4 *)(o + mt * 16) = acc[mt] * inv;
        }
        return;
    }

    // ---- split mode: merge the wavefronts through LDS. Rows are D+4 floats apart so that the sixteen
    // lanes of a row group write their 16-byte pieces to distinct banks.
    __syncthreads();
    float *mg = (float *)lds;
    constexpr int RS = D + 4;                 // padded row stride (floats)
    constexpr int WSTRIDE = 16 * RS + 32;     // one wavefront's slot: acc[16][RS], m[16], l[16]
    {
        float *w = mg + wave * WSTRIDE;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) *(f32x4 *)(w + n * RS + mt * 16 + g * 4) = acc[mt];
        if (g == 0) { w[16 * RS + n] = m_run; w[16 * RS + 16 + n] = l_run; }
    }
    __syncthreads();
    // every thread derives the weights exp2(m_w - m_all) of its own row from the NW maxima (NW LDS reads that
    // the sixteen lanes of a row share, NW exp2): cheaper than a serial pass by sixteen threads and a third barrier
    // partial slot layout in global memory (read by attn_merge_kernel): [16][D] o, [16] m, [16] l
    constexpr int PSTRIDE = 16 * D + 32;
    const size_t pslot = ((size_t)(unit * a.row_tiles + rt) * a.nseg + seg) * PSTRIDE;
    for (int e = threadIdx.x; e < 16 * D / 4; e += NW * 64) {
        const int row = e / (D / 4), col = (e % (D / 4)) * 4;
        float mw[NW];
        float m_all = -INFINITY;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            mw[w] = mg[w * WSTRIDE + 16 * RS + row];
            m_all = fmaxf(m_all, mw[w]);
        }
        f32x4 o = f32x4{0.f, 0.f, 0.f, 0.f};
        float l_all = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const float f = mw[w] > -INFINITY ? exp2f((mw[w] - m_all) * LOG2E) : 0.f;
            l_all += mg[w * WSTRIDE + 16 * RS + 16 + row] * f;
            o += *(const f32x4 *)(mg + w * WSTRIDE + row * RS + col) * f;
        }
        if (a.nseg == 1) {
            const int rr = rt * 16 + row;
            if (rr < a.rows_total) {
                const int l2 = rr / a.groups, g2 = rr % a.groups;
                const float inv = l_all > 0.f ? 1.f / l_all : 0.f;
                *(f32x4 *)(a.out + (((size_t)b * a.L + l2) * a.Hq + hk * a.groups + g2) * D + col) = o * inv;
            }
        } else {
            *(f32x4 *)(a.partial + pslot + row * D + col) = o;
            if (col == 0) {
                a.partial[pslot + 16 * D + row] = m_all;
                a.partial[pslot + 16 * D + 16 + row] = l_all;
            }
        }
    }
}

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
constexpr int PF_ROWS = 128, PF_TK = 64, PF_VROW = 136;
constexpr float PF_LAZY = 8.f;
#ifndef PF_AHEAD
#define PF_AHEAD 3
#endif
#ifndef PF_FLASH_BELOW
#define PF_FLASH_BELOW 8   // prompts whose 128-row workgroups would fill under 1/PF_FLASH_BELOW of the CUs run on the 16-row split kernel
#endif
#ifndef PF_SEG_TILES
#define PF_SEG_TILES 4     // fewest 64-key tiles a key segment of the prefill kernel is worth
#endif
#ifndef PF_PIPE_D
#define PF_PIPE_D 256      // head sizes from here on run the software-pipelined tile loop
#endif
using f32x16 = __attribute__((ext_vector_type(16))) float;
using u32x2 = __attribute__((ext_vector_type(2))) unsigned int;

template <int D>
struct PrefillCfg {
    static constexpr int KROW = D * 2;                              // unpadded (filled by LDS-writing loads), chunk slots swizzled
    static constexpr int K_BYTES = PF_TK * KROW;
    static constexpr int V_BYTES = D * PF_VROW;
    static constexpr int STAGE = K_BYTES + V_BYTES;
    static constexpr int LDS_BYTES = 2 * STAGE + 64;
};

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
    float *part = nullptr;
    if (nseg > 1) part = a.partial + ((size_t)(unit * a.row_tiles + (r >> 4)) * nseg + seg) * (16 * D + 32);
    if (nothing) {                                      // nothing visible to any row: zeros / an empty partial
        if (row_ok) {
            float *o = nseg > 1 ? part + (r & 15) * D : a.out + qbase;
            for (int d = lh * (D / 2); d < (lh + 1) * (D / 2); d += 4) *(f32x4 *)(o + d) = f32x4{0.f, 0.f, 0.f, 0.f};
            if (nseg > 1 && lh == 0) {
                part[16 * D + (r & 15)] = -INFINITY;
                part[16 * D + 16 + (r & 15)] = 0.f;
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
        // anyway, and a branch around the MFMAs makes the compiler carry the accumulators in vector registers
        // and copy all of them to and from the accumulation registers on every tile.
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
            if (__any(alpha != 1.f)) {              // wavefront-uniform and rare: must stay a branch, not a select
                // The accumulators live in accumulation registers for the MFMAs. Written as plain C++ the multiply
                // makes the compiler keep them in vector registers around this branch and copy all of them back and
                // forth on the common path (several hundred moves per key tile). So: read, scale and write back each
                // one here, with the register class pinned. The s_nops cover the waits between an MFMA result and
                // its read, and between the write-back and the next MFMA, which the compiler cannot see in here.
                asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");
#pragma unroll
                for (int j = 0; j < NJ; ++j)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        float tmp;
                        asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 1\n\tv_accvgpr_write_b32 %0, %1"
                                     : "+a"(acc[j][i]), "=&v"(tmp) : "v"(alpha));
                    }
                asm volatile("s_nop 7" ::: "memory");
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
    // operand addresses: K row (kb*32 + l31) at slot (2*kk + lh) ^ swz(row); V^T row (j*32 + l31), keys of step s2
    const int k_swz = CPK >= 16 ? (l31 & 15) : ((l31 >> 1) & 7);
    const int k_row = l31 * Cfg::KROW;
    const int v_off = Cfg::K_BYTES + l31 * PF_VROW + lh * 8;        // + j * 32 rows + s2 * 32 bytes (+16 for the second 4 keys)

    // Head size 256 and up (below, the serial loop above is faster: fewer MFMAs per tile to hide anything behind).
    // The loop is software-pipelined over the key tiles: iteration t computes S_t = K_t . Q^T, then the softmax of
    // S_t (vector ALU) TOGETHER WITH O += V_(t-1)^T . P_(t-1) (matrix pipe) - one wavefront per SIMD has nobody else
    // to fill the matrix pipe while it computes exponentials, so it has to overlap the two itself. P_(t-1) and the
    // running statistics of tile t-1 are consistent with the accumulators; the rescale by alpha_t follows the product.
    // LDS: K_t sits in stage t&1 (requested an iteration ahead), V_t is requested into registers in iteration t-1,
    // transposed into stage t&1 at the top of iteration t and consumed in iteration t+1: one barrier per tile.
    f32x16 sc[2];
    u32x4 pf[4] = {};
    auto tile_qk = [&](const unsigned char *st) __attribute__((always_inline)) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int i = 0; i < 16; ++i) sc[kb][i] = 0.f;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) {
            const int slot = ((2 * kk + lh) ^ k_swz) * 16;
            const u32x4 k0 = *(const u32x4 *)(st + k_row + slot);
            const u32x4 k1 = *(const u32x4 *)(st + 32 * Cfg::KROW + k_row + slot);
            sc[0] = mfma32<KV>(k0, qf[kk], sc[0]);
            sc[1] = mfma32<KV>(k1, qf[kk], sc[1]);
        }
    };
    // scaled (capped, masked) scores of the tile: lane holds keys key0 + kb*32 + (i/4)*8 + lh*4 + i%4 of row l31.
    // No branch in this kernel may contain an MFMA on the output accumulators (the compiler would then carry them in
    // vector registers and copy all of them to and from the accumulation registers on every tile), so the one
    // wavefront-uniform branch of a tile - mask or no mask - sits here, around vector instructions only.
    float x[32];
    auto tile_scores = [&](int key0) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            float v = sc[i >> 4][i & 15] * a.scale;
            if (CAP) v = a.soft_cap * tanhf(v * cap_inv);
            x[i] = v;
        }
        const bool full = key0 >= w_lo_max && key0 + PF_TK <= w_hi_min;   // every key visible to every row
        if (!full) {
            // key = key0 + 4*lh + c_i is visible iff lo <= key < hi, i.e. (unsigned)(c_i - lo_rel) < span
            const int lo_rel = lo - (key0 + lh * 4);
            const unsigned span = (unsigned)(hi - lo);
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                const int c = (i >> 4) * 32 + ((i >> 2) & 3) * 8 + (i & 3);
                x[i] = (unsigned)(c - lo_rel) < span ? x[i] : -INFINITY;
            }
        }
    };
    // softmax of x -> pf (next iteration's P^T operand), interleaved with the product of the previous tile
    auto tile_softmax_pv = [&](auto with_pv_c, const unsigned char *vst) __attribute__((always_inline)) {
        constexpr bool WITH_PV = decltype(with_pv_c)::value;
        // The softmax is cut into 32 units of a few vector instructions, and the product of the previous tile into its
        // NM MFMAs; unit group k is issued right behind MFMA k and a scheduling barrier keeps the pairs in this order
        // (left to itself the compiler issues the whole softmax first and the MFMAs behind it). The V^T operand of
        // MFMA k + PV_AHEAD is requested behind MFMA k.
        //   units 0..7    partial maxima of four scores each (two chains)
        //   unit  8       row maximum across the two lane halves, new reference maximum, alpha, exponent offset
        //   units 9..24   two exponentials each, partial sums (two chains)
        //   units 25..28  the four P^T operands of the next product
        //   unit  29      row sum across the lane halves, running sum and maximum
        constexpr int NM = 4 * NJ, UPM = 32 / NM, PV_AHEAD = NM >= 16 ? 4 : 2;
        float mxp[2] = {-INFINITY, -INFINITY}, rs[2] = {0.f, 0.f};
        float m_new = m_run, alpha = 1.f, mneg = 0.f;
        u32x4 pn[4];
        auto unit = [&](int u) __attribute__((always_inline)) {
            if (u < 8) {
                mxp[u & 1] = fmaxf(fmaxf(mxp[u & 1], fmaxf(x[4 * u], x[4 * u + 1])), fmaxf(x[4 * u + 2], x[4 * u + 3]));
            } else if (u == 8) {
                float mx = fmaxf(mxp[0], mxp[1]);
                mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
                // the reference maximum only moves when the tile's maximum exceeds it by more than PF_LAZY:
                // probabilities stay below e^PF_LAZY (exact in the f32 sums, fine in the 16-bit operand) and the
                // 2*D-register rescale of the accumulators becomes rare after the first tiles
                m_new = mx > m_run + PF_LAZY ? mx : m_run;
                // branch-free: with nothing visible so far (m_new = -inf) the exponent's offset is 0 and every
                // masked score still gives exp2(-inf) = 0
                alpha = m_run > -INFINITY ? __builtin_amdgcn_exp2f((m_run - m_new) * LOG2E) : 1.f;
                mneg = m_new > -INFINITY ? -m_new * LOG2E : 0.f;
            } else if (u < 25) {
                const int i0 = 2 * (u - 9);
                x[i0] = __builtin_amdgcn_exp2f(fmaf(x[i0], LOG2E, mneg));
                x[i0 + 1] = __builtin_amdgcn_exp2f(fmaf(x[i0 + 1], LOG2E, mneg));
                rs[0] += x[i0];
                rs[1] += x[i0 + 1];
            } else if (u < 29) {
                const int s2 = u - 25;
                // P^T operand of 16-key step s2: slots 0..7 <- accumulator elements 8*s2 .. 8*s2+7
                pn[s2] = u32x4{pack2<KV>(x[8 * s2], x[8 * s2 + 1]), pack2<KV>(x[8 * s2 + 2], x[8 * s2 + 3]),
                               pack2<KV>(x[8 * s2 + 4], x[8 * s2 + 5]), pack2<KV>(x[8 * s2 + 6], x[8 * s2 + 7])};
            } else if (u == 29) {
                float rowsum = rs[0] + rs[1];
                rowsum += __shfl_xor(rowsum, 32, 64);
                l_run = l_run * alpha + rowsum;
                m_run = m_new;
            }
        };
        if (WITH_PV) {
            // -- O^T += V^T . P^T of the previous tile; key step outermost: consecutive MFMAs go to different accumulators
            auto v_operand = [&](int idx) __attribute__((always_inline)) {
                const unsigned char *vrow = vst + v_off + (idx % NJ) * 32 * PF_VROW + (idx / NJ) * 32;
                const u32x2 va = *(const u32x2 *)(vrow), vb = *(const u32x2 *)(vrow + 16);
                return u32x4{va.x, va.y, vb.x, vb.y};
            };
            u32x4 vop[PV_AHEAD];
#pragma unroll
            for (int k = 0; k < PV_AHEAD; ++k) vop[k] = v_operand(k);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int k = 0; k < NM; ++k) {
                acc[k % NJ] = mfma32<KV>(vop[k % PV_AHEAD], pf[k / NJ], acc[k % NJ]);
                if (k + PV_AHEAD < NM) vop[k % PV_AHEAD] = v_operand(k + PV_AHEAD);
#pragma unroll
                for (int u = k * UPM; u < (k + 1) * UPM; ++u) unit(u);
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
#pragma unroll
            for (int u = 0; u < 30; ++u) unit(u);
        }
        if (__any(alpha != 1.f)) {              // wavefront-uniform and rare: must stay a branch, not a select
            // The accumulators live in accumulation registers for the MFMAs. Written as plain C++ the multiply
            // makes the compiler keep them in vector registers around this branch and copy all of them back and
            // forth on the common path (several hundred moves per key tile). So: read, scale and write back each
            // one here, with the register class pinned. The s_nops cover the waits between an MFMA result and
            // its read, and between the write-back and the next MFMA, which the compiler cannot see in here.
            asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    float tmp;
                    asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 1\n\tv_accvgpr_write_b32 %0, %1"
                                 : "+a"(acc[j][i]), "=&v"(tmp) : "v"(alpha));
                }
            asm volatile("s_nop 7" ::: "memory");
        }
#pragma unroll
        for (int s2 = 0; s2 < 4; ++s2) pf[s2] = pn[s2];
    };
    auto pin_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int i = 0; i < 16; ++i) asm volatile("" : "+a"(acc[j][i]));
    };
    using yes = std::integral_constant<bool, true>;
    using no = std::integral_constant<bool, false>;

    // one tile's front half: V_t to LDS for the next iteration's product, requests for tile t+1, S_t
    auto tile_front = [&](int t) __attribute__((always_inline)) {
        unsigned char *st = lds + ((t - t_begin) & 1) * Cfg::STAGE;
        unsigned char *other = lds + ((t - t_begin + 1) & 1) * Cfg::STAGE;
        store_v(st);
        // unconditional (a branch would split the block): past the end the last tile is requested once more, into
        // the stage and the registers that nobody reads again
        const int tn = min(t + 1, t_end - 1);
        load_k(tn, other);
        load_v(tn);
        tile_qk(st);
        // issue order: the LDS reads run PF_AHEAD k-steps ahead of the MFMAs that consume them (left alone the
        // compiler issues each read right before its MFMA, which then waits out the whole LDS latency)
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * PF_AHEAD, 0);
#pragma unroll
        for (int kk = 0; kk < KK - PF_AHEAD; ++kk) {
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 2 * PF_AHEAD, 0);
        tile_scores(t * PF_TK);
    };

    load_k(t_begin, lds);
    load_v(t_begin);
    __syncthreads();                                               // K of the first tile has landed (fence)
    // first tile, peeled: there is no previous product to overlap with
    tile_front(t_begin);
    tile_softmax_pv(no{}, lds);
    __syncthreads();
    for (int t = t_begin + 1; t < t_end; ++t) {
        // the accumulators are declared to sit in accumulation registers here and after the front half: without
        // these two pins the register allocator parks them in vector registers while S_t is computed and copies all
        // of them back for the product (2 x D/2 moves per tile)
        pin_acc();
        tile_front(t);
        pin_acc();
        tile_softmax_pv(yes{}, lds + ((t - t_begin + 1) & 1) * Cfg::STAGE);
        __syncthreads();                                           // also waits for this wavefront's K loads (fence)
    }
    {   // the last tile's product
        const unsigned char *vst = lds + ((t_end - 1 - t_begin) & 1) * Cfg::STAGE;
        constexpr int NM = 4 * NJ, PV_AHEAD = 4;
        auto v_operand = [&](int idx) __attribute__((always_inline)) {
            const unsigned char *vrow = vst + v_off + (idx % NJ) * 32 * PF_VROW + (idx / NJ) * 32;
            const u32x2 va = *(const u32x2 *)(vrow), vb = *(const u32x2 *)(vrow + 16);
            return u32x4{va.x, va.y, vb.x, vb.y};
        };
        u32x4 vop[PV_AHEAD];
#pragma unroll
        for (int k = 0; k < PV_AHEAD; ++k) vop[k] = v_operand(k);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k = 0; k < NM; ++k) {
            acc[k % NJ] = mfma32<KV>(vop[k % PV_AHEAD], pf[k / NJ], acc[k % NJ]);
            if (k + PV_AHEAD < NM) vop[k % PV_AHEAD] = v_operand(k + PV_AHEAD);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    }

    if (row_ok) {
        const float inv = nseg > 1 ? 1.f : (l_run > 0.f ? 1.f / l_run : 0.f);          // empty interval -> zeros
        float *o = nseg > 1 ? part + (r & 15) * D : a.out + qbase;
        if (nseg > 1 && lh == 0) {
            part[16 * D + (r & 15)] = m_run;
            part[16 * D + 16 + (r & 15)] = l_run;
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
    float m_loc = -INFINITY, l_loc = 0.f;
    f32x4 o_loc = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int s0 = sg; s0 < a.nseg; s0 += MERGE_SG * MERGE_UNROLL) {
        float ms[MERGE_UNROLL], ls[MERGE_UNROLL];
        f32x4 os[MERGE_UNROLL];
#pragma unroll
        for (int u = 0; u < MERGE_UNROLL; ++u) {
            const int sidx = min(s0 + u * MERGE_SG, a.nseg - 1);      // clamped: every load is unconditional
            const float *p = base + (size_t)sidx * WSTRIDE;
            ms[u] = p[16 * D + row];
            ls[u] = p[16 * D + 16 + row];
            os[u] = *(const f32x4 *)(p + row * D + dv);
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

// The same merge for many rows and few segments (the prefill kernel's key segments): one thread per (row, four
// consecutive dv), so that a wavefront reads whole contiguous rows of every segment's accumulators.
template <int D>
__global__ __launch_bounds__(256) void attn_merge_rows_kernel(AttnArgs a) {
    constexpr int WSTRIDE = 16 * D + 32;
    constexpr int TPR = D / 4, RPB = 256 / TPR;          // threads per row, rows per workgroup
    constexpr int UN = 4;
    const int unit = blockIdx.y, b = unit / a.Hkv, hk = unit % a.Hkv;
    const int rr = blockIdx.x * RPB + (int)threadIdx.x / TPR, dv = ((int)threadIdx.x % TPR) * 4;
    if (rr >= a.rows_total) return;
    const int rt = rr >> 4, row = rr & 15;
    const float *base = a.partial + (size_t)(unit * a.row_tiles + rt) * a.nseg * WSTRIDE;
    float m_all = -INFINITY, l_all = 0.f;
    f32x4 o = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < a.nseg; s0 += UN) {
        float ms[UN], ls[UN];
        f32x4 os[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const float *p = base + (size_t)min(s0 + u, a.nseg - 1) * WSTRIDE;      // clamped: every load is unconditional
            ms[u] = p[16 * D + row];
            ls[u] = p[16 * D + 16 + row];
            os[u] = *(const f32x4 *)(p + row * D + dv);
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
    const bool split = a.rows_total <= 64 || (!HILO && (long)units * ((a.rows_total + PF_ROWS - 1) / PF_ROWS) * PF_FLASH_BELOW <= cus0);
    if (split) {
        // key segments: one 32-key tile per wavefront while that leaves the device under-filled,
        // more tiles per wavefront beyond one workgroup per CU (its LDS tiles fill a CU)
        const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
        const int tiles = (a.T + TILE_KEYS - 1) / TILE_KEYS;
        int nseg = (cus + units * a.row_tiles - 1) / (units * a.row_tiles);
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
        using PCfg = PrefillCfg<D>;
        // No more workgroups than CUs: the key range of every row tile is cut into segments (at least
        // PF_SEG_TILES tiles each) and the partial results are merged, as in the decode path. Measured at 8 heads
        // x head size 256: L = 4096 (256 workgroups) 167 -> 136 us with two segments, L = 3072 125 -> 90 us.
        const int wgs = units * ((a.rows_total + PF_ROWS - 1) / PF_ROWS);
        const int key_tiles = (a.T + PF_TK - 1) / PF_TK;
        int want = cus0 / max(wgs, 1);
        if (want < 2 && wgs <= cus0) want = 2;      // one round of workgroups: two segments even out what a causal mask skews
        int nseg = max(1, min(min(want, key_tiles / PF_SEG_TILES), 16));
        a.nseg = nseg;
        if (nseg > 1) {
            const size_t bytes = (size_t)units * a.row_tiles * nseg * (16 * D + 32) * sizeof(float);
            int rc = ensure_scratch2(ctx, bytes);
            if (rc) return rc;
            a.partial = (float *)ctx->scratch2;
        }
        static bool attr_pf[2] = {false, false};
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
            launch_k(ctx, attn_merge_rows_kernel<D>, dim3((unsigned)((a.rows_total + RPB - 1) / RPB), (unsigned)units), dim3(256), 0, a);
        }
        LAUNCH_CHECK(ctx, "attn_prefill");
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
