// The 16-row flash attention body (split mode: a decode or a short prompt; per-wavefront mode: the hi+lo precise path over
// many rows), shared by attn_flash_kernel (attention.hip) and the one-launch decoder stack (decode_stack.hip), which runs
// it as one phase of a longer kernel with the queries arriving late and the output going to its exchange buffers. The
// formulation is described at the top of attention.hip.
#pragma once
#include "attention_common.h"

namespace attn {

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
template <int KV, int D, bool SPLIT, bool HILO, bool RING, class Hooks>
__device__ __forceinline__ void attn_flash_body(const AttnArgs &a, unsigned char *lds, const int block_x, const int block_y, Hooks &hooks) {
    const int ring = RING ? a.ring : 0;
    constexpr int NW = SPLIT ? SPLIT_NW : 4;
    using Cfg = FlashCfg<D, NW>;
    constexpr int KK = D / 32;   // MFMA k-steps over the head dim
    constexpr int MT = D / 16;   // 16-wide dv tiles

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = lane & 15, g = lane >> 4;
    const int unit = block_y;
    const int b = unit / a.Hkv, hk = unit % a.Hkv;
    int rt, seg;
    if (SPLIT) { rt = block_x / a.nseg; seg = block_x % a.nseg; }
    else { rt = block_x * 4 + wave; seg = 0; }

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
    if (q_shared && Hooks::Q_LATE) {
        // the queries are not there yet (they arrive while the first K/V tile is in flight): hooks.late_q below
    } else if (q_shared) {
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
    // Tile layout: key row of D*2 bytes, 16-byte chunk c of key k at slot c ^ (2 * ((k >> 2) & 3)) ^ (8 * (k & 1)) (the
    // last term for rows of 256 bytes and more; 128-byte rows alternate bank halves by themselves): the sixteen keys
    // one transposing read of the second product covers (four key groups x four keys) then fall on eight distinct
    // 32-byte bank ranges, two keys each - 512 bytes in the two passes they need anyway. Keys outside the union interval are read from
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
    (void)NVI; (void)KEYS_PER_VI; (void)vb8; (void)v_key_in; (void)v_slot; (void)v_hi_key;   // (used by the V loads, which exist in the device pass only)
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
            const int chunk = v_slot ^ (2 * grp) ^ (D >= 128 ? 8 * (key & 1) : 0);
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
    // V^T operand addresses (second product): lane = 16*g + 4*r + q reads key 4g+r (and 16+4g+r), dv 16*mt + 4q .. +3
    const int tr_r = (lane >> 2) & 3, tr_q = lane & 3;
    const unsigned v_rowaddr = (unsigned)(size_t)(lds_void *)vs + (unsigned)((4 * g + tr_r) * Cfg::ROW_BYTES + (tr_q & 1) * 8);
    const unsigned v_slot_l = (unsigned)(((tr_q >> 1) ^ (2 * g) ^ (D >= 128 ? 8 * (tr_r & 1) : 0)) << 4);
    if (t_begin < t_end) {
        load_k(t_begin);
        load_v(t_begin);
    }
    if (q_shared) {
        unsigned char *qsm = lds + Cfg::Q_OFF;
        if (Hooks::Q_LATE) {
            const int r2 = rt * 16 + qs_row;
            const bool live = qs_row < 16 && rt < a.row_tiles && r2 < a.rows_total;
            hooks.late_q(live ? (((size_t)b * a.L + r2 / a.groups) * a.Hq + hk * a.groups + r2 % a.groups) * D + qs_col : (size_t)0, live, qs0, qs1);
        }
        if (qs_row < 16)
            *(u32x4 *)(qsm + qs_row * Cfg::Q_ROW + qs_col * 2) =
                u32x4{pack2<KV>(qs0.x, qs0.y), pack2<KV>(qs0.z, qs0.w), pack2<KV>(qs1.x, qs1.y), pack2<KV>(qs1.z, qs1.w)};
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) qf[kk] = *(const u32x4 *)(qsm + n * Cfg::Q_ROW + kk * 64 + g * 16);
    }
    if constexpr (Hooks::Q_LATE) {
        // The first tile was requested before the caller's late operands arrived; a key row written since then (the row a
        // decode step appends) is stale in it. K: the lane that holds that key takes the row from the caller instead.
        const int rel = hooks.new_key() - t_begin * TILE_KEYS;
        if (t_begin < t_end && rel >= 0 && rel < TILE_KEYS && n == (rel & 15)) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
                if (h == (rel >> 4)) {
#pragma unroll
                    for (int kk = 0; kk < KK; ++kk) kf[h][kk] = hooks.new_k(hk * D + kk * 32 + g * 8);
                }
        }
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
        if constexpr (Hooks::Q_LATE) {
            // V: the same stale row, overwritten in the wavefront's LDS tile (16-byte chunk c of key k sits in slot
            // c ^ 2 * ((k >> 2) & 3) ^ 8 * (k & 1), the last term for rows of 256 bytes and more) before any operand read
            const int rel = hooks.new_key() - key0;
            if (t == t_begin && rel >= 0 && rel < TILE_KEYS && lane < D / 8) {
                const int slot = lane ^ (2 * ((rel >> 2) & 3)) ^ (D >= 128 ? 8 * (rel & 1) : 0);
                *(u32x4 *)(vs + rel * Cfg::ROW_BYTES + slot * 16) = hooks.new_v(hk * D + lane * 8);
            }
        }

        // -- O^T += V^T . P^T ; operand slot j of lane group g is key g*4+j (j<4) / 16+g*4+j-4
        const bool rescale = __any(alpha != 1.f);     // wavefront-uniform: skip 4*MT multiplies when no row's max moved
        // The V^T operand of a 16-dv tile comes by two transposing LDS reads (ds_read_b64_tr_b16: within 16 lanes, lane
        // 4r+q supplies the address of 4 consecutive dv of key r, lane i receives keys 0..3 of dv i): keys 4g+r and
        // 16+4g+r of row-major V, dv 16*mt + 4q .. +3, which is the slot order above. Written as assembly and waited for
        // by count: as a builtin the compiler would wait for every load in flight - the next tile's K - before the first.
        constexpr int VA = 2;                                        // operands requested ahead
        u32x4 vop[VA];
        auto v_operand = [&](auto mt_c) __attribute__((always_inline)) {
            constexpr int mt = decltype(mt_c)::value;
            const unsigned addr = v_rowaddr + (v_slot_l ^ (unsigned)(mt << 5));
            u32x2 a0, a1;
            asm volatile("ds_read_b64_tr_b16 %0, %2\n\tds_read_b64_tr_b16 %1, %2 offset:%3"
                         : "=&v"(a0), "=&v"(a1) : "v"(addr), "n"(16 * Cfg::ROW_BYTES) : "memory");
            return u32x4{a0.x, a0.y, a1.x, a1.y};
        };
        static_for<0, VA>([&](auto mc) __attribute__((always_inline)) { vop[decltype(mc)::value] = v_operand(mc); });
        static_for<0, MT>([&](auto mc) __attribute__((always_inline)) {
            constexpr int mt = decltype(mc)::value;
            constexpr int later = MT - 1 - mt < VA - 1 ? MT - 1 - mt : VA - 1;
            asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(vop[mt % VA]) : "n"(2 * later));
            f32x4 c = acc[mt];
            if (rescale) c *= alpha;
            c = mfma16<KV>(vop[mt % VA], pf, c);
            if (HILO) c = mfma16<KV>(vop[mt % VA], pf_lo, c);
            acc[mt] = c;
            if constexpr (mt + VA < MT) vop[mt % VA] = v_operand(std::integral_constant<int, mt + VA>{});
        });
        if (more) load_v(t + t_step);      // the operand reads above are complete: each was waited for before its MFMA
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
                hooks.store_out(a.out, (((size_t)b * a.L + l2) * a.Hq + hk * a.groups + g2) * D + col, o * inv);
            }
        } else if (rt * 16 + row < a.rows_total) {        // (rows past the last query row are padding: nobody reads them)
            *(f32x4 *)(a.partial + pslot + row * D + col) = o;
            if (col == 0) {
                a.partial[pslot + 16 * D + row] = m_all;
                a.partial[pslot + 16 * D + 16 + row] = l_all;
            }
        }
    }
}

}  // namespace attn
