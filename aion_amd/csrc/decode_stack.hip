// One launch for every transformer block of a single-token decode step.
//
// aion's Session.execute receives the whole ExecutableProgram (backend/backend.zig:42-44); for a decoder the program
// repeats one block per layer (src/bench/models.zig:433-536): RMSNorm -> MatMul q,k,v -> RoPE1D -> Cast f16 +
// SequenceAppend -> Attention -> MatMul o (+ residual) -> RMSNorm -> MatMul gate,up -> gate(gelu) -> MatMul down
// (+ residual). As separate launches every one of those steps sits on a dispatch floor of a few microseconds while the
// layer's weights would stream in under five, so here the whole run of blocks is ONE kernel of co-resident workgroups
// (one per CU, launched cooperatively) that walks the layers phase by phase:
//   P1  x -> RMSNorm -> int8 preparation -> q,k,v rows -> RoPE            (every workgroup, a few rows each)
//   P2  the new k,v rows -> f16 cache; attention over the cache            (one workgroup per kv head and row tile)
//   P3  attention output -> int8 preparation -> o rows + residual          (every workgroup)
//   P4  x -> RMSNorm -> preparation -> gate,up rows -> gelu*up -> preparation of the gated block
//   P5  prepared gated row -> down rows + residual
// Between phases a small vector (2048 ... 10240 values) has to reach every workgroup. It travels as 64-bit words
// {f32 value, 32-bit tag}: a device-scope atomic store publishes value and validity together, consumers poll the words
// they need with device-scope atomic loads until every tag is the expected one. No barrier, no fence, no flag behind the
// data: one store trip and one load round trip per phase (about 2.4 us on MI355X). Tags are unique per (launch, layer,
// phase): the launch counter lives in device memory and a one-thread launch behind the kernel moves it on, so a replayed
// recording is valid too.
// A buffer written in phase p is rewritten one layer later; by then every reader has consumed it: a workgroup reads a
// phase's input only if it also produces in that phase (one without rows in a phase skips it), it reads ALL of the
// input before it publishes anything, and whoever rewrites the buffer has - through the phases in between - waited
// for the words of every such producer.
// Every poll is bounded by a wall-clock budget. On expiry (a launch that is not co-resident, a lost workgroup) the
// workgroup raises a device error flag and exits; the others see the flag in their own polls and exit as well, so the
// grid always drains. The host reads the flag with aionhip_decoder_stack_status.
// The weights of a phase are requested before its poll, so their HBM latency hides under the exchange.
// Arithmetic: the device functions of the separate steps' kernels (prepare_act_block8, the RMSNorm of
// rmsnorm_kernel's summation order, v_dot4 block dots folded by wave_sum, rope_rotate, aion_gate_gelu, the flash
// attention body of attention_flash.h with one key tile per wavefront pass) in the same order per output, so a step
// gives the bits of the launch-per-step schedule as long as the cache holds at most 256 tokens (beyond that the
// separate attention step cuts the keys into segments that a second launch merges; here the eight wavefronts of one
// workgroup walk all tiles - the same sums in another order).
#include "attention_flash.h"

#include <algorithm>
#include <cmath>
#include <new>

namespace {
using namespace attn;

constexpr int DS_NT = 512;              // threads per workgroup: the eight wavefronts of the attention body's split shape
constexpr int DS_NW = DS_NT / 64;
using u64 = unsigned long long;

struct DsLayer {
    const u32x4 *wq, *wk, *wv, *wo, *wg, *wu, *wd;      // codes, device row layout
    const __half *sq, *sk, *sv, *so, *sg, *su, *sd;     // block scales
    const float *g1, *b1, *g2, *b2;                     // RMSNorm gamma / beta (beta may be null)
    __half *kc, *vc;                                    // caches [t_cap][h_kv][d] f16
};

struct DsArgs {
    const DsLayer *layers;
    int n_layers, hidden, heads, kv_heads, d, ffn, t_cap, rope_pairs;
    float eps1, eps2, attn_scale, soft_cap;
    unsigned win_left, win_right, win_chunk;
    const float *freq;
    const float *x_in;
    float *x_out;
    const int *positions, *write_index, *kv_lengths;
    u64 *xw, *qkvw, *attw, *x1w, *hw;                  // exchange buffers
    unsigned *epoch;
    int *err;
    long long budget;                                   // wall-clock ticks a poll may take before the workgroup gives up
    const float *q_dummy;                               // a 16-byte aligned address for the attention body's (unused) q operand
    long long *stamps;                                  // diagnostics, usually null: [2 workgroups][layers][10] wall-clock readings
};

struct Poll {
    long long t0, budget;
    int *err;
    bool dead;
};

__device__ __forceinline__ void ll_store(u64 *p, unsigned tag, unsigned bits) {
    __hip_atomic_store(p, ((u64)tag << 32) | (u64)bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Collects words [0, n) of `src` into dst (their value halves) once each carries `tag`. Every thread owns words
// tid, tid + NT, ...; MAXW of them are requested together and asked for again until all are valid. (Two requests in
// flight half a round trip apart were measured: the doubled poll traffic of 256 workgroups slowed every exchange down.)
template <int MAXW>
__device__ __forceinline__ void ll_gather(const u64 *src, int n, unsigned tag, unsigned *dst, Poll &pc) {
    const int tid = threadIdx.x;
    for (int base = 0; base < n; base += DS_NT * MAXW) {
        u64 w[MAXW];
        int spins = 0;
        while (true) {
#pragma unroll
            for (int j = 0; j < MAXW; ++j) w[j] = __hip_atomic_load(src + min(base + j * DS_NT + tid, n - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            bool ok = true;
#pragma unroll
            for (int j = 0; j < MAXW; ++j) ok = ok && (base + j * DS_NT + tid >= n || (unsigned)(w[j] >> 32) == tag);
            if (ok || pc.dead) break;
            if (pc.budget == 0 || (++spins & 15) == 0) {       // (a budget of zero gives up at the first poll that finds a word missing)
                if (wall_clock64() - pc.t0 >= pc.budget || __hip_atomic_load(pc.err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) pc.dead = true;
            }
        }
#pragma unroll
        for (int j = 0; j < MAXW; ++j)
            if (base + j * DS_NT + tid < n) dst[base + j * DS_NT + tid] = (unsigned)w[j];
    }
}

// R weight rows of one wavefront: base addresses of their codes and scales
template <int R>
struct Rows {
    const u32x4 *q[R];
    const __half *s[R];
};

// requests the first PRE 16-byte chunks of every row for this lane (clamped addresses: the loads are unconditional)
template <int DT, int R, int PRE>
__device__ __forceinline__ void rows_preload(const Rows<R> &rw, int lane, int chunks, u32x4 (&w)[PRE][R], __half (&hs)[PRE][R]) {
    constexpr bool Q8 = DT == AIONHIP_Q8_0;
#pragma unroll
    for (int u = 0; u < PRE; ++u) {
        const int ch = min(lane + 64 * u, chunks - 1);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            w[u][r] = __builtin_nontemporal_load(rw.q[r] + ch);
            hs[u][r] = rw.s[r][Q8 ? (ch >> 1) : ch];
        }
    }
}

// The block dots of R rows against the prepared activation in LDS, lane l taking chunks l, l + 64, ... in order, then
// the fold over the wavefront: the order of gemv_fused_kernel / gemv_kernel, hence their bits.
template <int DT, int R, int PRE>
__device__ __forceinline__ void rows_dot(const Rows<R> &rw, int lane, int chunks, const u32x4 (&w0)[PRE][R], const __half (&hs0)[PRE][R],
                                         const u32x4 *aq, const float *s_scale, const int *s_sum, float (&acc)[R]) {
    constexpr bool Q8 = DT == AIONHIP_Q8_0;
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;
    auto consume = [&](int ch, const u32x4 (&w)[R], const __half (&hs)[R]) {
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
                acc[r] += (float)d * (as * __half2float(hs[r]));
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
                acc[r] += (float)d * (as * __half2float(hs[r]));
            }
        }
    };
#pragma unroll
    for (int u = 0; u < PRE; ++u)
        if (lane + 64 * u < chunks) consume(lane + 64 * u, w0[u], hs0[u]);
#pragma unroll 1
    for (int ch = lane + 64 * PRE; ch < chunks; ch += 64) {
        u32x4 w[R];
        __half hs[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            w[r] = __builtin_nontemporal_load(rw.q[r] + ch);
            hs[r] = rw.s[r][Q8 ? (ch >> 1) : ch];
        }
        consume(ch, w, hs);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = wave_sum(acc[r]);
}

// LDS of the matmul phases (the attention phase reuses the same bytes, see decode_stack_lds)
struct PhaseLds {
    int *aq;          // prepared codes, K bytes
    float *scale;     // K / 32
    int *sum;         // K / 32
    float *red;       // 16 floats
    float *h;         // 32 floats: one gated block
    float *x;         // the f32 activation as it arrived
};
__host__ __device__ inline size_t phase_x_offset(int kmax) { return ((size_t)kmax + (size_t)(kmax / 32) * 8 + 64 + 128 + 15) & ~(size_t)15; }
__host__ __device__ inline size_t phase_lds_bytes(int kmax, int xmax) { return phase_x_offset(kmax) + (size_t)xmax * 4; }
__device__ __forceinline__ PhaseLds phase_lds(unsigned char *lds, int kmax) {
    PhaseLds p;
    p.aq = (int *)lds;
    p.scale = (float *)(lds + kmax);
    p.sum = (int *)(lds + kmax + (kmax / 32) * 4);
    p.red = (float *)(lds + kmax + (kmax / 32) * 8);
    p.h = p.red + 16;
    p.x = (float *)(lds + phase_x_offset(kmax));
    return p;
}

// int8 preparation of s.x[0, K) (PRO_QUANT of the one-row GEMV): codes, block scales, block code sums into LDS
__device__ __forceinline__ void prepare_plain(const PhaseLds &s, int K) {
    const int n4 = K >> 2;
    for (int c4 = threadIdx.x; c4 < ((n4 + 7) & ~7); c4 += DS_NT) {
        const bool live = c4 < n4;
        const f32x4 a = live ? *(const f32x4 *)(s.x + (size_t)c4 * 4) : f32x4{0.f, 0.f, 0.f, 0.f};
        int word, sq;
        float scale;
        prepare_act_block8(a.x, a.y, a.z, a.w, word, scale, sq);
        if (live) {
            s.aq[c4] = word;
            if ((c4 & 7) == 0) {
                s.scale[c4 >> 3] = scale;
                s.sum[c4 >> 3] = sq;
            }
        }
    }
}

// RMSNorm (aion cpu/exec/layernorm.zig:54-155) then the int8 preparation, as the PRO_RMSNORM prologue of the one-row
// GEMV computes them: the sum of squares is taken by 256 threads, thread t over float4 chunks t, t + 256, ... in
// order, folded per wavefront and then as (w0 + w1) + (w2 + w3).
// gm0 / bt0: gamma and beta of the thread's first chunk (c4 = tid), requested by the caller before it waited for x
__device__ __forceinline__ void prepare_rmsnorm(const PhaseLds &s, int K, const float *gamma, const float *beta, float eps, f32x4 gm0, f32x4 bt0) {
    const int tid = threadIdx.x, n4 = K >> 2;
    float ss = 0.f;
    if (tid < 256) {
        for (int c4 = tid; c4 < n4; c4 += 256) {
            const f32x4 v = *(const f32x4 *)(s.x + (size_t)c4 * 4);
            ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        }
    }
    ss = wave_sum(ss);
    if ((tid & 63) == 0 && tid < 256) s.red[tid >> 6] = ss;
    __syncthreads();
    const float tot = (s.red[0] + s.red[1]) + (s.red[2] + s.red[3]);
    const float inv_rms = 1.f / sqrtf(tot * (1.f / (float)K) + eps);
    for (int c4 = tid; c4 < ((n4 + 7) & ~7); c4 += DS_NT) {
        const bool live = c4 < n4;
        f32x4 a = f32x4{0.f, 0.f, 0.f, 0.f};
        if (live) {
            a = *(const f32x4 *)(s.x + (size_t)c4 * 4);
            const f32x4 gm = c4 == tid ? gm0 : *(const f32x4 *)(gamma + (size_t)c4 * 4);
            const f32x4 bt = c4 == tid ? bt0 : (beta ? *(const f32x4 *)(beta + (size_t)c4 * 4) : f32x4{0.f, 0.f, 0.f, 0.f});
            a.x = (a.x * inv_rms) * gm.x + bt.x;
            a.y = (a.y * inv_rms) * gm.y + bt.y;
            a.z = (a.z * inv_rms) * gm.z + bt.z;
            a.w = (a.w * inv_rms) * gm.w + bt.w;
        }
        int word, sq;
        float scale;
        prepare_act_block8(a.x, a.y, a.z, a.w, word, scale, sq);
        if (live) {
            s.aq[c4] = word;
            if ((c4 & 7) == 0) {
                s.scale[c4 >> 3] = scale;
                s.sum[c4 >> 3] = sq;
            }
        }
    }
}

// two tagged words with one 16-byte store (device scope: written through the XCD's L2). Each aligned 8-byte half is a
// complete {value, tag} word, so a reader that sees the halves at different times still never sees a torn word.
__device__ __forceinline__ void ll_store2(u64 *p, unsigned tag, unsigned b0, unsigned b1) {
    const u32x4 d{b0, tag, b1, tag};
    // (the wait state keeps the next instruction from overwriting the data registers while the store still reads them:
    // the compiler's hazard recognizer does not see through the assembly)
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(d) : "memory");
}

// The seams of the attention body inside this kernel: its first K/V tile is requested before the queries exist; late_q
// then waits for the block's q, k and v words, appends the new k and v rows to the f16 caches (aion cpu/exec/cast.zig,
// cpu/exec/sequence_append.zig:12-104) and hands the queries over from LDS; the appended row, stale in the tile
// requested earlier, is patched from LDS; the output rows leave as tagged words.
template <int D>
struct StackAttnHooks {
    static constexpr bool Q_LATE = true;
    const DsArgs &p;
    const DsLayer &L;
    float *qkv_f;              // LDS: q [heads * D], k [kv_heads * D], v [kv_heads * D] as they arrived
    unsigned tag_in, tag_out;
    int unit, rt, new_row;
    bool multi_tile;           // some wavefront walks more than one 32-key tile
    Poll &pc;
    long long q_at = 0;        // diagnostics: when the block's q, k and v had arrived
    bool dead = false;         // the wait for them ran out of time
    __device__ __forceinline__ void late_q(size_t index, bool live, f32x4 &q0, f32x4 &q1) {
        const int q_dim = p.heads * D, kv_dim = p.kv_heads * D;
        ll_gather<5>(p.qkvw, q_dim + 2 * kv_dim, tag_in, (unsigned *)qkv_f, pc);
        dead = __syncthreads_or(pc.dead ? 1 : 0) != 0;       // (the same for every thread; the caller leaves behind the body)
        if (p.stamps) q_at = wall_clock64();
        // this kv head's new rows -> the caches at the write index; only the first row tile's workgroup writes them
        if (rt == 0 && new_row >= 0) {
            for (int i = threadIdx.x; i < 2 * D; i += DS_NT) {
                const int which = i / D, e = i % D;
                __half *dst = (which == 0 ? L.kc : L.vc) + ((size_t)new_row * p.kv_heads + unit) * D + e;
                *dst = __float2half_rn(qkv_f[q_dim + which * kv_dim + unit * D + e]);
            }
        }
        // A wavefront that walks more than one key tile loads its later tiles from here on, and one of them may hold the
        // row: then the stores are complete before any such load. With at most one tile per wavefront (256 keys) nothing
        // is loaded any more and the wait is left out (the row reaches the tile in flight through the patch).
        if (multi_tile) {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        }
        if (live) {
            q0 = *(const f32x4 *)(qkv_f + index);
            q1 = *(const f32x4 *)(qkv_f + index + 4);
        }
    }
    __device__ __forceinline__ int new_key() { return new_row; }
    __device__ __forceinline__ u32x4 new_row_chunk(const float *src) {
        const f32x4 a = *(const f32x4 *)src, b = *(const f32x4 *)(src + 4);
        return u32x4{pack2<AIONHIP_F16>(a.x, a.y), pack2<AIONHIP_F16>(a.z, a.w), pack2<AIONHIP_F16>(b.x, b.y), pack2<AIONHIP_F16>(b.z, b.w)};
    }
    __device__ __forceinline__ u32x4 new_k(int off) { return new_row_chunk(qkv_f + p.heads * D + off); }
    __device__ __forceinline__ u32x4 new_v(int off) { return new_row_chunk(qkv_f + p.heads * D + p.kv_heads * D + off); }
    __device__ __forceinline__ void store_out(float *, size_t index, f32x4 v) {
        ll_store2(p.attw + index, tag_out, __float_as_uint(v.x), __float_as_uint(v.y));
        ll_store2(p.attw + index + 2, tag_out, __float_as_uint(v.z), __float_as_uint(v.w));
    }
};

__device__ __forceinline__ void stamp_at(const DsArgs &p, int stamp_wg, int l, int slot, long long t, int tid) {
    if (p.stamps && stamp_wg >= 0 && tid == 0) p.stamps[((size_t)stamp_wg * p.n_layers + l) * 10 + slot] = t;
}

// What a matmul wavefront keeps in registers from one block's attention phase on: the first chunks of the first row
// group of every matmul phase that follows (o, gate/up, down, the next block's q/k/v). They are requested while the
// attention runs and nothing waits for this workgroup, so that later every poll is alone in the wavefront's load queue
// (loads return in order: a poll issued behind a weight request would wait for the weights).
constexpr int PRE_O = 2, PRE_D = 4;
struct Prefetch {
    u32x4 w_gu[1][8], w_o[PRE_O][2], w_d[PRE_D][2];
    __half s_gu[1][8], s_o[PRE_O][2], s_d[PRE_D][2];
    f32x4 gm2, bt2;            // the second norm's gamma / beta chunk of this thread
    float res[2];              // the residuals of the wavefront's first two o rows
};

template <int DT, int D>
__global__ __launch_bounds__(DS_NT) void decode_stack_kernel(DsArgs p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    constexpr bool Q8 = DT == AIONHIP_Q8_0;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hidden = p.hidden, q_dim = p.heads * D, kv_dim = p.kv_heads * D, ffn = p.ffn;
    const unsigned epoch = *p.epoch;
    const unsigned tag0 = epoch * (unsigned)(p.n_layers * 8 + 8);
    Poll pc{wall_clock64(), p.budget, p.err, false};
    const int groups = p.heads / p.kv_heads;
    const int row_tiles = (groups + 15) / 16;
    const int attn_wgs = p.kv_heads * row_tiles;
    const int half = D >> 1;
    const bool is_attn = (int)blockIdx.x < attn_wgs;

    // a workgroup whose poll ran out of time raises the flag and leaves; every thread of the workgroup takes the same way
    auto gave_up = [&]() -> bool {
        const int any = __syncthreads_or(pc.dead ? 1 : 0);
        if (any && tid == 0) __hip_atomic_store(p.err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return any != 0;
    };
    // diagnostics: the first attention workgroup and the middle matmul workgroup note when each phase's input was complete
    // and when its output was out
    const int stamp_wg = blockIdx.x == 0 ? 0 : ((int)blockIdx.x == (int)gridDim.x / 2 ? 1 : -1);
    auto stamp = [&](int l, int slot) {
        if (p.stamps && stamp_wg >= 0 && tid == 0) p.stamps[((size_t)stamp_wg * p.n_layers + l) * 10 + slot] = wall_clock64();
    };

    // Work is dealt out over the matmul workgroups: the rows of all four matmuls. An attention workgroup only takes gate/up
    // blocks the matmul workgroups leave over (it is ahead of everyone at that point; o and down rows would make it late:
    // its polls would queue behind its own weight requests while everyone waits for its rows).
    const int n_g = (int)gridDim.x - attn_wgs;
    const int widx = is_attn ? n_g + (int)blockIdx.x : (int)blockIdx.x - attn_wgs;      // index among all workgroups, matmul ones first
    const int gw = widx * DS_NW + wave, total_waves = n_g * DS_NW;                       // rows: matmul workgroups only
    const int kmax = max(max(hidden, q_dim), ffn);
    const PhaseLds s = phase_lds(lds, kmax);
    const int ch_h = Q8 ? (hidden >> 4) : (hidden >> 5), ch_q = Q8 ? (q_dim >> 4) : (q_dim >> 5), ch_f = Q8 ? (ffn >> 4) : (ffn >> 5);
    const int kb_h = hidden >> 5, kb_q = q_dim >> 5, kb_f = ffn >> 5;
    const int per_head = D >> 3;
    const int tq = q_dim >> 3, tk = kv_dim >> 3, n_tasks1 = tq + 2 * tk, n_blocks = ffn >> 5;
    const bool has_p1 = !is_attn && widx * DS_NW < n_tasks1, has_rows = !is_attn && widx * DS_NW < hidden, has_p4 = widx < n_blocks;

    // row groups of the wavefront's tasks
    auto qkv_rows = [&](const DsLayer &L, int t, Rows<8> &rw, int &seg, int &row0) {
        // task t: rows head * D + e0 + {0..3} and head * D + D/2 + e0 + {0..3} (both halves of four RoPE pairs) of q, k or v
        seg = t < tq ? 0 : (t < tq + tk ? 1 : 2);
        const int tt = t - (seg == 0 ? 0 : (seg == 1 ? tq : tq + tk));
        row0 = (tt / per_head) * D + (tt % per_head) * 4;
        const u32x4 *qs = seg == 0 ? L.wq : (seg == 1 ? L.wk : L.wv);
        const __half *sc = seg == 0 ? L.sq : (seg == 1 ? L.sk : L.sv);
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const int row = row0 + (r & 3) + (r >> 2) * half;
            rw.q[r] = qs + (size_t)row * ch_h;
            rw.s[r] = sc + (size_t)row * kb_h;
        }
    };
    auto gu_rows = [&](const DsLayer &L, int blk, Rows<8> &rw) {
        const int r0 = blk * 32 + wave * 4;        // outputs r0 .. r0+3 of the gate (rows 0..3) and the up weight (rows 4..7)
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const int row = r0 + (r & 3);
            rw.q[r] = (r < 4 ? L.wg : L.wu) + (size_t)row * ch_h;
            rw.s[r] = (r < 4 ? L.sg : L.su) + (size_t)row * kb_h;
        }
    };
    auto two_rows = [&](const u32x4 *wq, const __half *wsc, int row_a, int row_b, int chunks, int kb, Rows<2> &rw) {
        rw.q[0] = wq + (size_t)row_a * chunks;
        rw.s[0] = wsc + (size_t)row_a * kb;
        rw.q[1] = wq + (size_t)row_b * chunks;
        rw.s[1] = wsc + (size_t)row_b * kb;
    };
    const int c4_own = min(tid, (hidden >> 2) - 1);      // the thread's first float4 chunk of a hidden-sized vector

    // Requests, for block l, what its o / gate,up / down phases will stream first and the small operands they need: all of
    // it is in flight while the attention runs (matmul workgroups) or right behind it (attention workgroups), so that
    // later every poll is alone in the wavefront's load queue.
    auto prefetch_tail = [&](int l, const DsLayer &L, Prefetch &pf) {
        const int row_a = min(gw, hidden - 1), row_b = min(gw + total_waves, hidden - 1);
        Rows<2> r2;
        two_rows(L.wo, L.so, row_a, row_b, ch_q, kb_q, r2);
        rows_preload<DT, 2, PRE_O>(r2, lane, ch_q, pf.w_o, pf.s_o);
        Rows<8> r8;
        gu_rows(L, min(widx, n_blocks - 1), r8);
        rows_preload<DT, 8, 1>(r8, lane, ch_h, pf.w_gu, pf.s_gu);
        two_rows(L.wd, L.sd, row_a, row_b, ch_f, kb_f, r2);
        rows_preload<DT, 2, PRE_D>(r2, lane, ch_f, pf.w_d, pf.s_d);
        pf.gm2 = *(const f32x4 *)(L.g2 + (size_t)c4_own * 4);
        pf.bt2 = L.b2 ? *(const f32x4 *)(L.b2 + (size_t)c4_own * 4) : f32x4{0.f, 0.f, 0.f, 0.f};
        // the residuals of the o rows: this block's input (its exchange words stay until the block's last phase rewrites
        // them; every word was valid before any q/k/v word of the block was written)
        pf.res[0] = l == 0 ? p.x_in[row_a] : __uint_as_float((unsigned)__hip_atomic_load(p.xw + row_a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
        pf.res[1] = l == 0 ? p.x_in[row_b] : __uint_as_float((unsigned)__hip_atomic_load(p.xw + row_b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    };

    // The three matmul phases behind the attention, for every workgroup. Returns false when the workgroup gave up.
    auto tail_phases = [&](int l, const DsLayer &L, Prefetch &pf) -> bool {
        const unsigned tag_x = tag0 + (unsigned)(l * 8), tag_att = tag_x + 2, tag_x1 = tag_x + 3, tag_h = tag_x + 4, tag_out = tag_x + 8;
        float x1_own[2] = {0.f, 0.f};            // the o rows this wavefront produced first: the residuals of its first down rows
        // ================= P3: o rows + residual =================
        if (has_rows) {
            ll_gather<4>(p.attw, q_dim, tag_att, (unsigned *)s.x, pc);
            if (gave_up()) return false;
            stamp(l, 4);
            prepare_plain(s, q_dim);
            __syncthreads();
            // a wavefront takes rows gw and gw + (wavefronts) together, then the next such pair; the first pair was requested
            // during the attention
            for (int row = gw; row < hidden; row += 2 * total_waves) {
                const int row_b = row + total_waves;
                Rows<2> rw;
                two_rows(L.wo, L.so, row, min(row_b, hidden - 1), ch_q, kb_q, rw);
                float res0 = pf.res[0], res1 = pf.res[1];
                if (row != gw) {
                    rows_preload<DT, 2, PRE_O>(rw, lane, ch_q, pf.w_o, pf.s_o);
                    res0 = l == 0 ? p.x_in[row] : __uint_as_float((unsigned)__hip_atomic_load(p.xw + row, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
                    res1 = l == 0 ? p.x_in[min(row_b, hidden - 1)]
                                  : __uint_as_float((unsigned)__hip_atomic_load(p.xw + min(row_b, hidden - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
                }
                float acc[2];
                rows_dot<DT, 2, PRE_O>(rw, lane, ch_q, pf.w_o, pf.s_o, (const u32x4 *)s.aq, s.scale, s.sum, acc);
                const float out0 = acc[0] + 1.f * res0, out1 = acc[1] + 1.f * res1;
                if (row == gw) { x1_own[0] = out0; x1_own[1] = out1; }
                if (lane == 0) {
                    ll_store(p.x1w + row, tag_x1, __float_as_uint(out0));
                    if (row_b < hidden) ll_store(p.x1w + row_b, tag_x1, __float_as_uint(out1));
                }
            }
            stamp(l, 5);
        }
        // ================= P4: RMSNorm -> gate, up rows -> gelu * up -> preparation of the gated block =================
        if (has_p4) {
            ll_gather<4>(p.x1w, hidden, tag_x1, (unsigned *)s.x, pc);
            if (gave_up()) return false;
            stamp(l, 6);
            prepare_rmsnorm(s, hidden, L.g2, L.b2, p.eps2, pf.gm2, pf.bt2);
            __syncthreads();
            for (int blk = widx; blk < n_blocks; blk += (int)gridDim.x) {
                Rows<8> rw;
                gu_rows(L, blk, rw);
                if (blk != widx) rows_preload<DT, 8, 1>(rw, lane, ch_h, pf.w_gu, pf.s_gu);
                float acc[8];
                rows_dot<DT, 8, 1>(rw, lane, ch_h, pf.w_gu, pf.s_gu, (const u32x4 *)s.aq, s.scale, s.sum, acc);
                if (lane < 4) {
                    const float gv = (lane == 0 ? acc[0] : lane == 1 ? acc[1] : lane == 2 ? acc[2] : acc[3]);
                    const float uv = (lane == 0 ? acc[4] : lane == 1 ? acc[5] : lane == 2 ? acc[6] : acc[7]);
                    s.h[wave * 4 + lane] = aion_gate_gelu(gv, uv);
                }
                __syncthreads();
                if (tid < 8) {
                    // the block's int8 preparation (aion cpu/kernels/matmul_q_i8.zig:187-203), 8 lanes x 4 values
                    const float v0 = s.h[tid * 4], v1 = s.h[tid * 4 + 1], v2 = s.h[tid * 4 + 2], v3 = s.h[tid * 4 + 3];
                    int word, sq;
                    float scale;
                    prepare_act_block8(v0, v1, v2, v3, word, scale, sq);
                    ll_store(p.hw + blk * 8 + tid, tag_h, (unsigned)word);
                    if (tid == 0) {
                        ll_store(p.hw + (ffn >> 2) + blk, tag_h, __float_as_uint(scale));
                        ll_store(p.hw + (ffn >> 2) + n_blocks + blk, tag_h, (unsigned)sq);
                    }
                }
                __syncthreads();                            // s.h is reused by the next block
            }
            stamp(l, 7);
        }
        // ================= P5: down rows + residual =================
        if (has_rows) {
            const bool last = l + 1 == p.n_layers;
            // the prepared gated row arrives as it is used: codes, block scales, block code sums
            ll_gather<5>(p.hw, (ffn >> 2) + 2 * kb_f, tag_h, (unsigned *)s.x, pc);
            if (gave_up()) return false;
            stamp(l, 8);
            for (int i = tid; i < (ffn >> 2) + 2 * kb_f; i += DS_NT) {
                const unsigned v = ((const unsigned *)s.x)[i];
                if (i < (ffn >> 2)) s.aq[i] = (int)v;
                else if (i < (ffn >> 2) + kb_f) s.scale[i - (ffn >> 2)] = __uint_as_float(v);
                else s.sum[i - (ffn >> 2) - kb_f] = (int)v;
            }
            __syncthreads();
            for (int row = gw; row < hidden; row += 2 * total_waves) {
                const int row_b = row + total_waves;
                Rows<2> rw;
                two_rows(L.wd, L.sd, row, min(row_b, hidden - 1), ch_f, kb_f, rw);
                float res0 = x1_own[0], res1 = x1_own[1];
                if (row != gw) {
                    rows_preload<DT, 2, PRE_D>(rw, lane, ch_f, pf.w_d, pf.s_d);
                    res0 = __uint_as_float((unsigned)__hip_atomic_load(p.x1w + row, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
                    res1 = __uint_as_float((unsigned)__hip_atomic_load(p.x1w + min(row_b, hidden - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
                }
                float acc[2];
                rows_dot<DT, 2, PRE_D>(rw, lane, ch_f, pf.w_d, pf.s_d, (const u32x4 *)s.aq, s.scale, s.sum, acc);
                if (lane == 0) {
                    const float out0 = acc[0] + 1.f * res0, out1 = acc[1] + 1.f * res1;
                    if (last) {
                        p.x_out[row] = out0;
                        if (row_b < hidden) p.x_out[row_b] = out1;
                    } else {
                        ll_store(p.xw + row, tag_out, __float_as_uint(out0));
                        if (row_b < hidden) ll_store(p.xw + row_b, tag_out, __float_as_uint(out1));
                    }
                }
            }
            stamp(l, 9);
            __syncthreads();                                // the next phase of this workgroup rewrites s.x and s.aq
        }
        return true;
    };

    // ============================ the attention workgroups ============================
    if (is_attn) {
        const int unit = (int)blockIdx.x / row_tiles, rt = (int)blockIdx.x % row_tiles;
        using Cfg = FlashCfg<D, SPLIT_NW>;
        float *qkv_f = (float *)(lds + Cfg::LDS_BYTES);
        const long wi = (long)p.write_index[0];
        const int new_row = wi >= 0 && wi < (long)p.t_cap ? (int)wi : -1;
        const bool multi_tile = min(max(p.kv_lengths[0], 0), p.t_cap) > SPLIT_NW * TILE_KEYS;
        for (int l = 0; l < p.n_layers; ++l) {
            const DsLayer &L = p.layers[l];
            bool hooks_dead = false;
            {
                AttnArgs a{};
                a.q = p.q_dummy;
                a.k = L.kc;
                a.v = L.vc;
                a.out = nullptr;
                a.positions = p.positions;
                a.kv_lengths = p.kv_lengths;
                a.partial = nullptr;
                a.B = 1; a.L = 1; a.T = p.t_cap; a.Hq = p.heads; a.Hkv = p.kv_heads; a.groups = groups;
                a.rows_total = groups; a.row_tiles = row_tiles; a.nseg = 1; a.ring = 0;
                a.q_dtype = AIONHIP_F32; a.kv_dtype = AIONHIP_F16;
                a.scale = p.attn_scale; a.soft_cap = p.soft_cap;
                a.win_left = p.win_left; a.win_right = p.win_right; a.win_chunk = p.win_chunk;
                StackAttnHooks<D> hooks{p, L, qkv_f, tag0 + (unsigned)(l * 8) + 1, tag0 + (unsigned)(l * 8) + 2, unit, rt, new_row, multi_tile, pc};
                stamp(l, 0);
                attn_flash_body<AIONHIP_F16, D, true, false, false>(a, lds, rt, unit, hooks);
                stamp(l, 1);
                if (hooks.q_at) stamp_at(p, stamp_wg, l, 2, hooks.q_at, tid);
                hooks_dead = hooks.dead;
            }
            // The body's LDS may be reused once every wavefront is through with it; nothing here waits for the output words
            // to be acknowledged (a fencing barrier would: they are written through to memory).
            __builtin_amdgcn_s_waitcnt(0xC07F);          // lgkmcnt(0) only
            __builtin_amdgcn_s_barrier();
            if (hooks_dead) {
                if (tid == 0) __hip_atomic_store(p.err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                return;
            }
            stamp(l, 3);
            Prefetch pf;
            prefetch_tail(l, L, pf);
            if (!tail_phases(l, L, pf)) return;
        }
        return;
    }

    // ============================ the matmul workgroups ============================
    // The wavefront's q/k/v row group is the same in every block, and so is its RoPE angle: sine and cosine once.
    int seg1 = 0, row01 = 0;
    float sn1 = 0.f, cs1 = 1.f;
    bool rot1 = false;
    {
        Rows<8> rw;
        qkv_rows(p.layers[0], min(gw, n_tasks1 - 1), rw, seg1, row01);
        if (lane < 4) {
            const int i = row01 % D + lane;
            rot1 = seg1 < 2 && i < p.rope_pairs;
            if (rot1) sincosf((float)p.positions[0] * p.freq[i], &sn1, &cs1);
        }
    }
    const int pos = p.positions[0];
    // the wavefront's q/k/v rows of the block to come: requested here for the first block, during the attention of the
    // block before for every later one (a request right in front of the poll would hold the poll's answer back behind it)
    u32x4 w_qkv[1][8];
    __half s_qkv[1][8];
    {
        Rows<8> rw;
        int seg, row0;
        qkv_rows(p.layers[0], min(gw, n_tasks1 - 1), rw, seg, row0);
        rows_preload<DT, 8, 1>(rw, lane, ch_h, w_qkv, s_qkv);
    }
    for (int l = 0; l < p.n_layers; ++l) {
        const DsLayer &L = p.layers[l];
        const unsigned tag_x = tag0 + (unsigned)(l * 8), tag_qkv = tag_x + 1;
        // ================= P1: RMSNorm -> q, k, v rows -> RoPE =================
        if (has_p1) {
            // (this wavefront's rows were requested during the previous block's attention; the norm's operands are small)
            const f32x4 gm1 = *(const f32x4 *)(L.g1 + (size_t)c4_own * 4);
            const f32x4 bt1 = L.b1 ? *(const f32x4 *)(L.b1 + (size_t)c4_own * 4) : f32x4{0.f, 0.f, 0.f, 0.f};
            // the block's input: the step's input for the first block, the previous block's output words after that
            if (l == 0) {
                for (int c4 = tid; c4 < (hidden >> 2); c4 += DS_NT) *(f32x4 *)(s.x + (size_t)c4 * 4) = *(const f32x4 *)(p.x_in + (size_t)c4 * 4);
            } else {
                ll_gather<4>(p.xw, hidden, tag_x, (unsigned *)s.x, pc);
            }
            if (gave_up()) return;               // (a barrier: s.x is complete)
            stamp(l, 0);
            prepare_rmsnorm(s, hidden, L.g1, L.b1, p.eps1, gm1, bt1);
            __syncthreads();
            for (int t = gw; t < n_tasks1; t += total_waves) {
                Rows<8> rw;
                int seg, row0;
                qkv_rows(L, t, rw, seg, row0);
                if (t != gw) rows_preload<DT, 8, 1>(rw, lane, ch_h, w_qkv, s_qkv);
                float acc[8];
                rows_dot<DT, 8, 1>(rw, lane, ch_h, w_qkv, s_qkv, (const u32x4 *)s.aq, s.scale, s.sum, acc);
                if (lane < 4) {
                    // lane e finishes pair e (aion cpu/kernels/rope.zig:20-98): the arithmetic of the fused q/k/v step
                    const float xl = (lane == 0 ? acc[0] : lane == 1 ? acc[1] : lane == 2 ? acc[2] : acc[3]);
                    const float xh = (lane == 0 ? acc[4] : lane == 1 ? acc[5] : lane == 2 ? acc[6] : acc[7]);
                    const int head = row0 / D, i = row0 % D + lane;
                    bool rot = rot1;
                    float sn = sn1, cs = cs1;
                    if (t != gw) {
                        rot = seg < 2 && i < p.rope_pairs;
                        sn = 0.f; cs = 1.f;
                        if (rot) sincosf((float)pos * p.freq[i], &sn, &cs);
                    }
                    float yl = xl, yh = xh;
                    if (rot) rope_rotate(xl, xh, sn, cs, yl, yh);
                    u64 *dst = p.qkvw + (seg == 0 ? 0 : (seg == 1 ? q_dim : q_dim + kv_dim)) + head * D + i;
                    ll_store(dst, tag_qkv, __float_as_uint(yl));
                    ll_store(dst + half, tag_qkv, __float_as_uint(yh));
                }
            }
            stamp(l, 1);
        }
        Prefetch pf;
        prefetch_tail(l, L, pf);
        if (has_p1 && l + 1 < p.n_layers) {
            Rows<8> rw;
            int seg, row0;
            qkv_rows(p.layers[l + 1], min(gw, n_tasks1 - 1), rw, seg, row0);
            rows_preload<DT, 8, 1>(rw, lane, ch_h, w_qkv, s_qkv);
        }
        if (!tail_phases(l, L, pf)) return;
    }
}

// The launch counter moves on in a launch of its own behind the stack's: only then has every workgroup read it.
__global__ void decode_stack_next_epoch(unsigned *epoch) { *epoch += 1; }

template <int D>
size_t decode_stack_lds(int hidden, int q_dim, int kv_dim, int ffn) {
    const int kmax = std::max(std::max(hidden, q_dim), ffn), xmax = std::max(std::max(hidden, q_dim), ffn / 4 + ffn / 16);
    const size_t phase = phase_lds_bytes(kmax, xmax);
    const size_t attn_bytes = (size_t)FlashCfg<D, SPLIT_NW>::LDS_BYTES + (size_t)(q_dim + 2 * kv_dim) * 4;
    return std::max(phase, attn_bytes);
}

}  // namespace

struct aionhip_decoder_stack {
    DsArgs args{};
    int dtype = 0;
    void *dev_layers = nullptr, *exchange = nullptr, *flags = nullptr;
    size_t lds = 0;
    int grid = 0;
    void *kernel = nullptr;
};

extern "C" {

int aionhip_decoder_stack_create(aionhip_ctx *ctx, const aionhip_decoder_stack_desc *d, const aionhip_decoder_stack_layer *layers, aionhip_decoder_stack **out) {
    if (!ctx || !d || !layers || !out) return AIONHIP_INVALID_ARGUMENT;
    *out = nullptr;
    if (ctx->capturing) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "decoder_stack_create allocates and cannot be recorded into a program");
    if (d->layers == 0 || d->layers > 4096) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "decoder stack: 1..4096 layers");
    const size_t hidden = d->hidden, hq = d->heads, hkv = d->kv_heads, hd = d->head_dim, ffn = d->ffn;
    if (hq == 0 || hkv == 0 || hq % hkv != 0 || hidden == 0 || ffn == 0 || d->t_cap == 0)
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "decoder stack: zero dimension, or heads not a multiple of kv heads");
    if (!(d->eps1 > 0.f) || !(d->eps1 < INFINITY) || !(d->eps2 > 0.f) || !(d->eps2 < INFINITY))
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "decoder stack: eps must be positive and finite");
    if (!(d->rope_base > 0.f) || !(d->rope_base < INFINITY) || !(d->rope_scale > 0.f) || !(d->rope_scale < INFINITY) || !(d->rope_proportion >= 0.f && d->rope_proportion <= 1.f))
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "decoder stack: RoPE base/scale must be positive and finite, proportion in [0,1]");
    // the shapes the one-launch form takes; anything else runs as separate steps
    if ((hd != 128 && hd != 256) || hidden % 32 != 0 || ffn % 32 != 0 || hidden > 8192 || hq * hd > 8192 || ffn > 32768 || hq / hkv > 16 || d->t_cap > 0x7FFFFFFFu ||
        d->rolling || !(d->attn_scale > 0.f))
        return set_err(ctx, AIONHIP_UNSUPPORTED, "decoder stack: needs head size 128 or 256, hidden and heads x head size <= 8192, ffn <= 32768 (multiples of 32), "
                                                 "at most 16 query heads per kv head, linear caches and a positive softmax scale");
    const size_t q_dim = hq * hd, kv_dim = hkv * hd;
    int dtype = 0;
    std::vector<DsLayer> host(d->layers);
    for (size_t l = 0; l < d->layers; ++l) {
        const aionhip_decoder_stack_layer &s = layers[l];
        const aionhip_weight *ws[7] = {s.wq, s.wk, s.wv, s.wo, s.w_gate, s.w_up, s.w_down};
        const size_t ns[7] = {q_dim, kv_dim, kv_dim, hidden, ffn, ffn, hidden}, ks[7] = {hidden, hidden, hidden, q_dim, hidden, hidden, ffn};
        for (int i = 0; i < 7; ++i) {
            if (!ws[i]) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "decoder stack: layer %zu: null weight", l);
            if (ws[i]->n != ns[i] || ws[i]->k != ks[i]) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "decoder stack: layer %zu: weight %d is %zu x %zu, expected %zu x %zu", l, i, ws[i]->n, ws[i]->k, ns[i], ks[i]);
            if (l == 0 && i == 0) dtype = ws[i]->dtype;
            if (ws[i]->dtype != dtype) return set_err(ctx, AIONHIP_UNSUPPORTED, "decoder stack: all weights must share one block format");
            if (dtype != AIONHIP_Q4_0 && dtype != AIONHIP_Q8_0) return set_err(ctx, AIONHIP_UNSUPPORTED, "decoder stack: q4_0 or q8_0 weights only");
        }
        if (!s.norm1_gamma || !s.norm2_gamma || !s.k_cache || !s.v_cache) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "decoder stack: layer %zu: null gamma or cache", l);
        if ((s.norm1_gamma | s.norm1_beta | s.norm2_gamma | s.norm2_beta | s.k_cache | s.v_cache) & 15)
            return set_err(ctx, AIONHIP_UNSUPPORTED, "decoder stack: gamma, beta and the caches must be 16-byte aligned");
        DsLayer &o = host[l];
        o.wq = (const u32x4 *)s.wq->qs; o.wk = (const u32x4 *)s.wk->qs; o.wv = (const u32x4 *)s.wv->qs; o.wo = (const u32x4 *)s.wo->qs;
        o.wg = (const u32x4 *)s.w_gate->qs; o.wu = (const u32x4 *)s.w_up->qs; o.wd = (const u32x4 *)s.w_down->qs;
        o.sq = s.wq->sc; o.sk = s.wk->sc; o.sv = s.wv->sc; o.so = s.wo->sc; o.sg = s.w_gate->sc; o.su = s.w_up->sc; o.sd = s.w_down->sc;
        o.g1 = (const float *)(uintptr_t)s.norm1_gamma; o.b1 = (const float *)(uintptr_t)s.norm1_beta;
        o.g2 = (const float *)(uintptr_t)s.norm2_gamma; o.b2 = (const float *)(uintptr_t)s.norm2_beta;
        o.kc = (__half *)(uintptr_t)s.k_cache; o.vc = (__half *)(uintptr_t)s.v_cache;
    }
    aionhip_decoder_stack *st = new (std::nothrow) aionhip_decoder_stack();
    if (!st) return set_err(ctx, AIONHIP_OUT_OF_MEMORY, "host allocation failed");
    st->dtype = dtype;
    const bool q8 = dtype == AIONHIP_Q8_0;
    if (hd == 256) {
        st->kernel = q8 ? (void *)decode_stack_kernel<AIONHIP_Q8_0, 256> : (void *)decode_stack_kernel<AIONHIP_Q4_0, 256>;
        st->lds = decode_stack_lds<256>((int)hidden, (int)q_dim, (int)kv_dim, (int)ffn);
    } else {
        st->kernel = q8 ? (void *)decode_stack_kernel<AIONHIP_Q8_0, 128> : (void *)decode_stack_kernel<AIONHIP_Q4_0, 128>;
        st->lds = decode_stack_lds<128>((int)hidden, (int)q_dim, (int)kv_dim, (int)ffn);
    }
    auto fail = [&](int rc) {
        aionhip_decoder_stack_destroy(ctx, st);
        return rc;
    };
    if (st->lds > 160 * 1024) return fail(set_err(ctx, AIONHIP_UNSUPPORTED, "decoder stack: the shape needs %zu bytes of LDS per workgroup", st->lds));
    hipError_t e = hipFuncSetAttribute(st->kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)st->lds);
    if (e != hipSuccess) return fail(set_err(ctx, AIONHIP_EXECUTION_FAILED, "decoder stack: hipFuncSetAttribute: %s", hipGetErrorString(e)));
    int per_cu = 0;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, st->kernel, DS_NT, st->lds);
    if (e != hipSuccess || per_cu < 1) return fail(set_err(ctx, AIONHIP_UNSUPPORTED, "decoder stack: a %d-thread workgroup with %zu bytes of LDS does not fit a CU", DS_NT, st->lds));
    st->grid = ctx->cu_count > 0 ? ctx->cu_count : 256;
    if (st->grid < (int)(hkv * ((hq / hkv + 15) / 16))) return fail(set_err(ctx, AIONHIP_UNSUPPORTED, "decoder stack: more kv heads than CUs"));

    int rc = dev_malloc(ctx, &st->dev_layers, host.size() * sizeof(DsLayer), "decoder stack layers");
    if (rc) return fail(rc);
    // exchange words: x, q|k|v, attention output, x1, prepared gated row; then the launch counter and the error flag
    const size_t words = hidden + (q_dim + 2 * kv_dim) + q_dim + hidden + (ffn / 4 + 2 * (ffn / 32));
    rc = dev_malloc(ctx, &st->exchange, words * sizeof(u64), "decoder stack exchange");
    if (rc) return fail(rc);
    rc = dev_malloc(ctx, &st->flags, 256, "decoder stack flags");
    if (rc) return fail(rc);
    e = hipMemcpyAsync(st->dev_layers, host.data(), host.size() * sizeof(DsLayer), hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipMemsetAsync(st->exchange, 0, words * sizeof(u64), ctx->stream);
    if (e == hipSuccess) e = hipMemsetAsync(st->flags, 0, 256, ctx->stream);
    const unsigned one = 1;
    if (e == hipSuccess) e = hipMemcpyAsync(st->flags, &one, sizeof one, hipMemcpyHostToDevice, ctx->stream);   // launch counter: tag 0 is "never written"
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return fail(set_err(ctx, AIONHIP_EXECUTION_FAILED, "decoder stack set-up: %s", hipGetErrorString(e)));

    const size_t halfd = hd / 2;
    size_t rope_pairs = (size_t)floorf(d->rope_proportion * (float)halfd);
    if (rope_pairs > halfd) rope_pairs = halfd;
    const float freq_step = (float)pow((double)d->rope_base, (double)(-2.0f / (float)hd));
    const float *freq = nullptr;
    rc = rope_table(ctx, (int)rope_pairs, freq_step, d->rope_scale, &freq);
    if (rc) return fail(rc);

    DsArgs &a = st->args;
    a.layers = (const DsLayer *)st->dev_layers;
    a.n_layers = (int)d->layers; a.hidden = (int)hidden; a.heads = (int)hq; a.kv_heads = (int)hkv; a.d = (int)hd; a.ffn = (int)ffn;
    a.t_cap = (int)d->t_cap; a.rope_pairs = (int)rope_pairs;
    a.eps1 = d->eps1; a.eps2 = d->eps2; a.attn_scale = d->attn_scale; a.soft_cap = d->attn_logits_soft_cap;
    a.win_left = d->window_left; a.win_right = d->window_right; a.win_chunk = d->window_chunk;
    a.freq = freq;
    u64 *xw = (u64 *)st->exchange;
    a.xw = xw; a.qkvw = a.xw + hidden; a.attw = a.qkvw + (q_dim + 2 * kv_dim); a.x1w = a.attw + q_dim; a.hw = a.x1w + hidden;
    a.epoch = (unsigned *)st->flags;
    a.err = (int *)st->flags + 16;
    a.q_dummy = (const float *)st->exchange;
    int wall_khz = 0;
    if (hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, ctx->device) != hipSuccess || wall_khz <= 0) wall_khz = 100000;
    a.budget = (long long)wall_khz * 250;                 // 250 ms: a step takes well under one
    *out = st;
    return AIONHIP_OK;
}

void aionhip_decoder_stack_destroy(aionhip_ctx *ctx, aionhip_decoder_stack *st) {
    if (!st) return;
    if (ctx) (void)hipStreamSynchronize(ctx->stream);
    if (st->dev_layers) (void)hipFree(st->dev_layers);
    if (st->exchange) (void)hipFree(st->exchange);
    if (st->flags) (void)hipFree(st->flags);
    delete st;
}

int aionhip_decoder_stack_set_stamps(aionhip_ctx *ctx, aionhip_decoder_stack *st, aionhip_handle stamps) {
    if (!ctx || !st) return AIONHIP_INVALID_ARGUMENT;
    if (stamps & 7) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "decoder stack: the stamp buffer must be 8-byte aligned");
    st->args.stamps = (long long *)(uintptr_t)stamps;
    return AIONHIP_OK;
}

int aionhip_decoder_stack_set_poll_budget(aionhip_ctx *ctx, aionhip_decoder_stack *st, double milliseconds) {
    if (!ctx || !st) return AIONHIP_INVALID_ARGUMENT;
    if (!(milliseconds >= 0.0) || milliseconds > 10000.0) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "decoder stack: poll budget must be 0..10000 ms");
    int wall_khz = 0;
    if (hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, ctx->device) != hipSuccess || wall_khz <= 0) wall_khz = 100000;
    st->args.budget = (long long)((double)wall_khz * milliseconds);
    return AIONHIP_OK;
}

int aionhip_step_decoder_stack(aionhip_ctx *ctx, aionhip_decoder_stack *st, aionhip_handle x_in, aionhip_handle x_out,
                               aionhip_handle positions, aionhip_handle write_index, aionhip_handle kv_lengths) {
    if (!ctx || !st) return AIONHIP_INVALID_ARGUMENT;
    if (!x_in || !x_out || !positions || !write_index || !kv_lengths) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "decoder stack: null operand");
    if ((x_in & 15) || (x_out & 3) || ((positions | write_index | kv_lengths) & 3)) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "decoder stack: x_in must be 16-byte aligned, the others 4-byte aligned");
    DsArgs a = st->args;
    a.x_in = (const float *)(uintptr_t)x_in;
    a.x_out = (float *)(uintptr_t)x_out;
    a.positions = (const int *)(uintptr_t)positions;
    a.write_index = (const int *)(uintptr_t)write_index;
    a.kv_lengths = (const int *)(uintptr_t)kv_lengths;
    void *params[] = {&a};
    const char *name = st->dtype == AIONHIP_Q8_0 ? "decoder_stack_q8" : "decoder_stack_q4";
    hipEvent_t e0 = nullptr, e1 = nullptr;
    const bool timed = ctx->profiling && !ctx->capturing;
    if (timed) {
        ProfScope scope(ctx, name);
        prof_open(ctx, &e0, &e1);
        HIP_TRY(ctx, hipEventRecord(e0, ctx->stream));
    }
    // cooperative: the launch is refused, rather than left to wait for itself, when the grid cannot be resident at once
    HIP_TRY(ctx, hipLaunchCooperativeKernel(st->kernel, dim3((unsigned)st->grid), dim3(DS_NT), params, (unsigned)st->lds, ctx->stream));
    if (timed) HIP_TRY(ctx, hipEventRecord(e1, ctx->stream));
    decode_stack_next_epoch<<<dim3(1), dim3(1), 0, ctx->stream>>>(a.epoch);
    LAUNCH_CHECK(ctx, name);
    return AIONHIP_OK;
}

int aionhip_decoder_stack_status(aionhip_ctx *ctx, aionhip_decoder_stack *st, int *failed) {
    if (!ctx || !st || !failed) return AIONHIP_INVALID_ARGUMENT;
    if (ctx->capturing) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "decoder_stack_status synchronises and cannot be recorded into a program");
    int flag = 0;
    HIP_TRY(ctx, hipMemcpyAsync(&flag, st->args.err, sizeof flag, hipMemcpyDeviceToHost, ctx->stream));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    *failed = flag;
    if (flag) {
        // a launch gave up: its exchange words may hold tags of a step that never completed. Start over from a clean state.
        const size_t words = (size_t)st->args.hidden * 2 + (size_t)st->args.heads * st->args.d * 2 + (size_t)st->args.kv_heads * st->args.d * 2 +
                             (size_t)(st->args.ffn / 4 + 2 * (st->args.ffn / 32));
        HIP_TRY(ctx, hipMemsetAsync(st->exchange, 0, words * sizeof(u64), ctx->stream));
        HIP_TRY(ctx, hipMemsetAsync(st->args.err, 0, sizeof(int), ctx->stream));
        HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
        return set_err(ctx, AIONHIP_EXECUTION_FAILED, "decoder stack: a workgroup waited longer than the poll budget for another one's results (the grid was not "
                                                      "resident at once, or the device is shared); the step's outputs are invalid");
    }
    return AIONHIP_OK;
}

}  // extern "C"
