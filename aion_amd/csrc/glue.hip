// Per-token glue steps between the matmuls of a decoder: RMSNorm(+residual), RoPE, add,
// gelu-gate, row gather, f32->f16 cast + KV append, argmax. All HBM/launch-bound, one pass each.
// Formulas follow aion's CPU executors (cited per kernel) including its polynomial tanh/exp for
// the gelu gate, so a decoder run tracks the CPU path closely.
#include "common.h"

namespace {

// cpu/exec/layernorm.zig:54-155 + cpu/kernels/layernorm.zig:69-147 (rmsnorm mode):
// inv = 1/sqrt(sum(x^2)/cols + eps); out = (x*inv)*gamma + beta; out += residual
__global__ __launch_bounds__(256) void rmsnorm_kernel(float *out, const float *__restrict__ x, const float *__restrict__ gamma,
                                                      const float *__restrict__ beta, const float *residual,   // out may be residual
                                                      size_t cols, float eps) {
    __shared__ float red[4];
    const size_t row = blockIdx.x;
    const float *xr = x + row * cols;
    float ss = 0.f;
    for (size_t c = threadIdx.x; c < cols; c += 256) ss += xr[c] * xr[c];
    ss = block_sum_256(ss, red);
    const float inv = 1.f / sqrtf(ss * (1.f / (float)cols) + eps);
    for (size_t c = threadIdx.x; c < cols; c += 256) {
        float y = (xr[c] * inv) * gamma[c] + (beta ? beta[c] : 0.f);
        if (residual) y += residual[row * cols + c];
        out[row * cols + c] = y;
    }
}

// Rows of up to 2048 columns: the row, gamma, beta and the residual are all requested before the reduction, at clamped
// addresses without branches, so the step is one memory round trip and not two (a single-row launch is a chain of
// dependent latencies: 6.4 -> 3.6 us at 2048 columns). The sums run in rmsnorm_kernel's order: the same bits.
__global__ __launch_bounds__(256) void rmsnorm_short_kernel(float *out, const float *x, const float *__restrict__ gamma,
                                                            const float *__restrict__ beta, const float *residual, size_t cols, float eps) {
    __shared__ float red[4];
    const size_t row = blockIdx.x;
    const float *xr = x + row * cols;
    const float *rr = residual ? residual + row * cols : xr;
    const float *br = beta ? beta : gamma;
    float xv[8], gv[8], bv[8], rv[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const size_t c = min((size_t)threadIdx.x + 256 * j, cols - 1);
        xv[j] = xr[c];
        gv[j] = gamma[c];
        bv[j] = br[c];
        rv[j] = rr[c];
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j)
        if ((size_t)threadIdx.x + 256 * j < cols) ss += xv[j] * xv[j];
    ss = block_sum_256(ss, red);
    const float inv = 1.f / sqrtf(ss * (1.f / (float)cols) + eps);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const size_t c = (size_t)threadIdx.x + 256 * j;
        if (c >= cols) break;
        float y = (xv[j] * inv) * gv[j] + (beta ? bv[j] : 0.f);
        if (residual) y += rv[j];
        out[row * cols + c] = y;
    }
}

// cpu/exec/rope.zig:14-53 + cpu/kernels/rope.zig:20-98: pairs (i, i + D/2); the frequency is
// multiplied up iteratively in f32 (a per-context table built on the host) and the angle pos*f is
// rounded to f32, as on the CPU. aion takes sin/cos of that f32 angle in f64 and rounds; here
// sincosf (full range reduction, <= 2 ulp).

__global__ void rope_kernel(float *__restrict__ out, const float *__restrict__ x, const int *__restrict__ positions,
                            size_t tokens, int H, int D, int rope_pairs, const float *__restrict__ freq) {
    const int half = D / 2;
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= tokens * (size_t)half) return;
    const size_t tok = gid / half;
    const int i = (int)(gid % half);
    const float *xr = x + tok * H * D;
    float *orow = out + tok * H * D;
    if (i >= rope_pairs) {
        for (int h = 0; h < H; ++h) {
            orow[h * D + i] = xr[h * D + i];
            orow[h * D + half + i] = xr[h * D + half + i];
        }
        return;
    }
    const float ang = (float)positions[tok] * freq[i];
    float sn, cs;
    sincosf(ang, &sn, &cs);
    for (int h = 0; h < H; ++h) {
        const float xl = xr[h * D + i], xh = xr[h * D + half + i];
        rope_rotate(xl, xh, sn, cs, orow[h * D + i], orow[h * D + half + i]);
    }
}

// RoPE1D(q), RoPE1D(k) -> f16 -> SequenceAppend(k cache), Cast f16 + SequenceAppend(v cache) for the
// tokens of one step, as one launch: thread (token, head slot, pair i) rotates pair i of one q head,
// or of one k head (and copies the matching v elements). Same arithmetic as the four separate steps.
__global__ void rope_append_kernel(float *__restrict__ q_out, const float *__restrict__ q, const float *__restrict__ k, const float *__restrict__ v,
                                   __half *__restrict__ kcache, __half *__restrict__ vcache, const int *__restrict__ positions,
                                   const int *__restrict__ write_index, size_t batch, size_t s_len, size_t t_cap, int Hq, int Hkv, int D,
                                   int rope_pairs, const float *__restrict__ freq) {
    const int half = D / 2;
    const int slots = Hq + Hkv;
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= batch * s_len * (size_t)slots * half) return;
    const int i = (int)(gid % half);
    const int slot = (int)((gid / half) % slots);
    const size_t tok = gid / ((size_t)half * slots);          // b * s_len + s
    // every global operand is requested before the first use: one memory round trip
    const bool rot = i < rope_pairs;
    const bool is_q = slot < Hq;
    const int h = is_q ? slot : slot - Hq;
    const size_t src = is_q ? (tok * Hq + h) * D : (tok * Hkv + h) * D;
    const float *xp = is_q ? q : k;
    const int pos = positions[tok];
    const int widx = write_index[tok / s_len];                 // one write index per batch entry (sequence_append.zig:58-60)
    const float fr = i < rope_pairs ? freq[i] : 0.f;
    const float xl = xp[src + i], xh = xp[src + half + i];
    float vl = 0.f, vh = 0.f;
    if (!is_q) { vl = v[src + i]; vh = v[src + half + i]; }
    float sn = 0.f, cs = 1.f;
    if (rot) sincosf((float)pos * fr, &sn, &cs);
    float yl = xl, yh = xh;
    if (rot) rope_rotate(xl, xh, sn, cs, yl, yh);
    if (is_q) {
        q_out[src + i] = yl;
        q_out[src + half + i] = yh;
        return;
    }
    const size_t b = tok / s_len, s = tok % s_len;
    const long t = (long)widx + (long)s;
    if (t < 0 || (size_t)t >= t_cap) return;                   // never write outside the cache
    const size_t dst = ((b * t_cap + (size_t)t) * Hkv + h) * D;
    kcache[dst + i] = __float2half_rn(yl);
    kcache[dst + half + i] = __float2half_rn(yh);
    vcache[dst + i] = __float2half_rn(vl);
    vcache[dst + half + i] = __float2half_rn(vh);
}

// The input side of an attention block in a model that normalizes its heads (aion's bench model,
// src/bench/models.zig:455-473): RMSNorm over the head dimension on q, k and v (cpu/kernels/layernorm.zig:69-147), RoPE on
// q and k, f16 cast and cache append of k and v - eight to ten steps of a few microseconds each as one launch. One
// wavefront per (token, head): q heads first, then k, then v; lane l holds the pairs (i, i + D/2), i = l, l + 64, ...
__global__ __launch_bounds__(256) void headnorm_rope_append_kernel(
    float *__restrict__ q_out, const float *__restrict__ q, const float *__restrict__ k, const float *__restrict__ v,
    const float *__restrict__ gq, const float *__restrict__ bq, const float *__restrict__ gk, const float *__restrict__ bk,
    const float *__restrict__ gv, const float *__restrict__ bv, float eps, __half *__restrict__ kcache, __half *__restrict__ vcache,
    const int *__restrict__ positions, const int *__restrict__ write_index, size_t batch, size_t s_len, size_t t_cap, int Hq, int Hkv,
    int D, int rope_pairs, const float *__restrict__ freq, int rolling) {
    const int half = D / 2, slots = Hq + 2 * Hkv, lane = threadIdx.x & 63;
    const size_t item = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= batch * s_len * (size_t)slots) return;                     // wavefront-uniform
    const int slot = (int)(item % slots);
    const size_t tok = item / slots;
    const int kind = slot < Hq ? 0 : slot < Hq + Hkv ? 1 : 2;             // q, k, v
    const int h = kind == 0 ? slot : kind == 1 ? slot - Hq : slot - Hq - Hkv;
    const float *src = (kind == 0 ? q + (tok * Hq + h) * D : (kind == 1 ? k : v) + (tok * Hkv + h) * D);
    const float *gamma = kind == 0 ? gq : kind == 1 ? gk : gv, *beta = kind == 0 ? bq : kind == 1 ? bk : bv;
    const int pos = positions[tok];
    const int widx = write_index[tok / s_len];
    constexpr int MAXP = 4;                                                // pairs per lane: head sizes up to 512
    // everything the second half needs is requested here, at clamped addresses without branches, so that the launch is one
    // memory round trip: the row, gamma, beta and the rotation frequencies
    float xl[MAXP], xh[MAXP], gl[MAXP], gh[MAXP], bl[MAXP], bh[MAXP], fr[MAXP];
    const float *bsrc = beta ? beta : gamma;
#pragma unroll
    for (int u = 0; u < MAXP; ++u) {
        const int i = min(lane + 64 * u, half - 1);
        xl[u] = src[i];
        xh[u] = src[half + i];
        gl[u] = gamma[i];
        gh[u] = gamma[half + i];
        bl[u] = bsrc[i];
        bh[u] = bsrc[half + i];
        fr[u] = freq[rope_pairs > 0 ? min(i, rope_pairs - 1) : 0];
    }
    // the sum of squares in rmsnorm_kernel's order (thread c of 256 adds x[c]^2, x[c + 256]^2; four wavefront sums; their
    // pairwise sum), so that the fused step gives the bits of the separate ones: the row is read a second time, from L1
    float part[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int c = lane + 64 * j;
        float ssj = 0.f;
        if (c < D) ssj += src[c] * src[c];
        if (c + 256 < D) ssj += src[c + 256] * src[c + 256];
        part[j] = wave_sum(ssj);
    }
    const float ss = (part[0] + part[1]) + (part[2] + part[3]);
    const float inv = 1.f / sqrtf(ss * (1.f / (float)D) + eps);
    const size_t b = tok / s_len, s = tok % s_len;
    long t = (long)widx + (long)s;
    if (rolling && t >= 0) t %= (long)t_cap;
    const bool in_cache = t >= 0 && (size_t)t < t_cap;                     // never write outside the cache
    __half *dst = (kind == 1 ? kcache : vcache) + ((b * t_cap + (size_t)(in_cache ? t : 0)) * Hkv + h) * D;
#pragma unroll
    for (int u = 0; u < MAXP; ++u) {
        const int i = lane + 64 * u;
        if (i >= half) break;
        float yl = (xl[u] * inv) * gl[u] + (beta ? bl[u] : 0.f);
        float yh = (xh[u] * inv) * gh[u] + (beta ? bh[u] : 0.f);
        if (kind != 2 && i < rope_pairs) {
            float sn, cs;
            sincosf((float)pos * fr[u], &sn, &cs);
            rope_rotate(yl, yh, sn, cs, yl, yh);
        }
        if (kind == 0) {
            q_out[(tok * Hq + h) * D + i] = yl;
            q_out[(tok * Hq + h) * D + half + i] = yh;
        } else if (in_cache) {
            dst[i] = __float2half_rn(yl);
            dst[half + i] = __float2half_rn(yh);
        }
    }
}

__global__ void add_kernel(float *__restrict__ out, const float *__restrict__ a, const float *__restrict__ b, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = a[i] + b[i];
}

// cpu/exec/elementwise.zig:25-37 (gate) + cpu/kernels/gelu.zig:8-14
__global__ void gate_gelu_kernel(float *__restrict__ out, const float *__restrict__ a, const float *__restrict__ b, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    out[i] = aion_gate_gelu(a[i], b[i]);
}

// StepUnary on f32 (backend/types.zig:119-125, cpu/exec/unary.zig:55-64) with aion's exp-based approximations of
// sigmoid and tanh (cpu/kernels/fast_math.zig:53-148; gelu is the tanh form, cpu/kernels/gelu.zig:8-14)
template <int OP>
__global__ void unary_kernel(float *__restrict__ out, const float *__restrict__ x, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float v = x[i];
    float r;
    if (OP == AIONHIP_UNARY_RELU) r = v > 0.f ? v : 0.f;
    else if (OP == AIONHIP_UNARY_GELU) r = 0.5f * v * (1.f + aion_tanh_approx(0.7978845608028654f * (v + 0.044715f * (v * v * v))));
    else if (OP == AIONHIP_UNARY_SILU) r = v * aion_sigmoid_approx(v);
    else if (OP == AIONHIP_UNARY_SIGMOID) r = aion_sigmoid_approx(v);
    else if (OP == AIONHIP_UNARY_TANH) r = aion_tanh_approx(v);
    else r = sqrtf(v);
    out[i] = r;
}
// StepElemwiseBinary add / sub / mul / div on f32 where b has a's shape, is one element, or is a contiguous suffix of
// a's shape (cpu/exec/elementwise.zig:38-60: identical, scalar_b, contiguous_suffix_b): out[i] = a[i] op b[i % nb]
template <int OP>
__global__ void binary_kernel(float *__restrict__ out, const float *__restrict__ a, const float *__restrict__ b, size_t n, size_t nb) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float x = a[i], y = b[nb == n ? i : i % nb];
    out[i] = OP == AIONHIP_BINARY_ADD ? x + y : OP == AIONHIP_BINARY_SUB ? x - y : OP == AIONHIP_BINARY_MUL ? x * y : x / y;
}

// cpu/exec/gather.zig:60-87: one workgroup per gathered row; ids outside [0, vocab) give zeros
__global__ __launch_bounds__(256) void gather_rows_kernel(int dtype, float *__restrict__ out, const void *__restrict__ table,
                                                          const int *__restrict__ ids, size_t d, size_t vocab) {
    const size_t i = blockIdx.x;
    const long id = ids[i];
    float *o = out + i * d;
    if (id < 0 || (size_t)id >= vocab) {
        for (size_t c = threadIdx.x; c < d; c += 256) o[c] = 0.f;
        return;
    }
    if (dtype == AIONHIP_F32) {
        const float *src = (const float *)table + (size_t)id * d;
        for (size_t c = threadIdx.x; c < d; c += 256) o[c] = src[c];
    } else {
        const uint8_t *src = (const uint8_t *)table + (size_t)id * (d / QK) * Q8_BYTES;
        for (size_t c = threadIdx.x; c < d; c += 256) {
            const uint8_t *blk = src + (c / QK) * Q8_BYTES;
            const float s = __half2float(__ushort_as_half(*reinterpret_cast<const uint16_t *>(blk)));
            o[c] = (float)(int8_t)blk[2 + c % QK] * s;
        }
    }
}

// cpu/exec/cast.zig (f32 -> f16, RNE) and cpu/exec/sequence_append.zig:12-104
__global__ void cast_f16_kernel(__half *__restrict__ out, const float *__restrict__ x, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = __float2half_rn(x[i]);
}
// rolling: the cache is a ring, logical step t lives in row t % t_cap (storage/cache.zig:202-207)
__global__ void append_f16_kernel(__half *__restrict__ cache, const float *__restrict__ src, const int *__restrict__ write_index,
                                  size_t s_len, size_t t_cap, size_t row_elems, size_t total, int rolling) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const size_t e = i % row_elems, s = (i / row_elems) % s_len, b = i / (row_elems * s_len);
    long t = (long)write_index[b] + (long)s;      // one write index per batch entry (sequence_append.zig:58-60)
    if (t < 0) return;
    if (rolling) t %= (long)t_cap;
    if ((size_t)t >= t_cap) return;               // never write outside the cache
    cache[(b * t_cap + (size_t)t) * row_elems + e] = __float2half_rn(src[i]);
}
// StepSequenceAppend as the reference states it (cpu/exec/sequence_append.zig:12-104): rows and cache of one element type
template <typename T>
__global__ void append_same_kernel(T *__restrict__ cache, const T *__restrict__ src, const int *__restrict__ write_index,
                                   size_t s_len, size_t t_cap, size_t row_elems, size_t total, int rolling) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const size_t e = i % row_elems, s = (i / row_elems) % s_len, b = i / (row_elems * s_len);
    long t = (long)write_index[b] + (long)s;
    if (t < 0) return;
    if (rolling) t %= (long)t_cap;
    if ((size_t)t >= t_cap) return;
    cache[(b * t_cap + (size_t)t) * row_elems + e] = src[i];
}

// Growth of a sequence cache along its time axis (storage/manager/grow.zig:37-78): the wider backing is zero
// except for the `outer` preserved runs, each copied to the start of its wider slot. One pass over the new
// backing in 4-byte words (the reference's device path also moves whole words).
__global__ void cache_grow_kernel(unsigned *__restrict__ dst, const unsigned *__restrict__ src, size_t old_words, size_t new_words, size_t total) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const size_t o = i / new_words, r = i % new_words;
    dst[i] = r < old_words ? src[o * old_words + r] : 0u;
}
// The same for a ring (grow.zig:107-150): row t % capacity changes with the capacity, so the retained logical
// steps of batch entry b - the last min(end, retained_history, old_capacity) before end = logical_ends[b] - are
// re-placed; every other row of the new ring is zero. A new row p holds the step t = end-1 - ((end-1-p) mod
// new_capacity) if that step is retained (at most one retained step maps to a row, as kept <= old < new capacity).
__global__ void cache_grow_rolling_kernel(unsigned *__restrict__ dst, const unsigned *__restrict__ src, const int *__restrict__ logical_ends,
                                          size_t old_cap, size_t new_cap, size_t row_words, size_t retained, size_t total) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const size_t w = i % row_words, p = (i / row_words) % new_cap, b = i / (row_words * new_cap);
    const long end = logical_ends[b];
    unsigned v = 0u;
    if (end > 0) {
        const size_t e = (size_t)end;
        size_t kept = e < retained ? e : retained;
        if (old_cap < kept) kept = old_cap;
        const size_t last = e - 1;
        const size_t back = (last % new_cap + new_cap - p) % new_cap;      // steps from `last` back to the one living in row p
        if (back < kept) {
            const size_t t = last - back;
            v = src[(b * old_cap + t % old_cap) * row_words + w];
        }
    }
    dst[i] = v;
}

// cpu/exec/argmax.zig:56-81: strict > keeps the first maximum. ARGMAX_PARTS workgroups per row each reduce a contiguous
// slice to (value, index); the workgroup that draws the row's last ticket then picks among the parts (ties -> the smaller
// index, which is the first maximum) - one launch. A part travels as ONE 64-bit word {value bits, index}, stored and loaded
// as a single device-scope atomic, so a reader can never see the value of one store with the index of another; the ticket
// is a device-scope read-modify-write with release (the part's word is visible before the ticket counts it) and acquire
// (the last workgroup's loads of the parts are ordered behind its ticket) semantics. The pick does not depend on which
// workgroup came last. Tickets return to zero.
constexpr int ARGMAX_PARTS = 64;
__device__ __forceinline__ void argmax_reduce_256(float &best, int &idx, float *bv, int *bi) {
    bv[threadIdx.x] = best;
    bi[threadIdx.x] = idx;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) {
            const float ov = bv[threadIdx.x + s];
            const int oi = bi[threadIdx.x + s];
            if (oi != 0x7FFFFFFF && (bi[threadIdx.x] == 0x7FFFFFFF || ov > bv[threadIdx.x] || (ov == bv[threadIdx.x] && oi < bi[threadIdx.x]))) {
                bv[threadIdx.x] = ov;
                bi[threadIdx.x] = oi;
            }
        }
        __syncthreads();
    }
    best = bv[0];
    idx = bi[0];
    __syncthreads();
}
__global__ __launch_bounds__(256) void argmax_kernel(int *__restrict__ out, unsigned long long *parts, unsigned *tickets, const float *__restrict__ x, size_t n) {
    __shared__ float bv[256];
    __shared__ int bi[256];
    __shared__ int s_last;
    const size_t row = blockIdx.y;
    const size_t per = (n + ARGMAX_PARTS - 1) / ARGMAX_PARTS;
    const size_t lo = blockIdx.x * per, hi = lo + per < n ? lo + per : n;
    const float *r = x + row * n;
    float best = -INFINITY;
    int idx = 0x7FFFFFFF;
    for (size_t j = lo + threadIdx.x; j < hi; j += 256) {
        const float v = r[j];
        if (idx == 0x7FFFFFFF || v > best) { best = v; idx = (int)j; }
    }
    argmax_reduce_256(best, idx, bv, bi);
    if (threadIdx.x == 0) {
        const unsigned long long word = ((unsigned long long)__float_as_uint(best) << 32) | (unsigned)idx;
        __hip_atomic_store(parts + row * ARGMAX_PARTS + blockIdx.x, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = __hip_atomic_fetch_add(tickets + row, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT) == ARGMAX_PARTS - 1;
    }
    __syncthreads();
    if (!s_last) return;
    best = -INFINITY;
    idx = 0x7FFFFFFF;
    if (threadIdx.x < ARGMAX_PARTS) {
        const unsigned long long word = __hip_atomic_load(parts + row * ARGMAX_PARTS + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        best = __uint_as_float((unsigned)(word >> 32));
        idx = (int)(unsigned)word;
    }
    argmax_reduce_256(best, idx, bv, bi);
    if (threadIdx.x == 0) {
        out[row] = idx == 0x7FFFFFFF ? 0 : idx;
        __hip_atomic_store(tickets + row, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

inline unsigned grid_for(size_t n, unsigned block) { return (unsigned)((n + block - 1) / block); }
template <class T>
inline T *dp(aionhip_handle h) { return (T *)(uintptr_t)h; }

}  // namespace

int launch_rmsnorm(aionhip_ctx *ctx, float *out, const float *x, const float *gamma, const float *beta, const float *residual,
                   size_t rows, size_t cols, float eps) {
    if (cols <= 2048) rmsnorm_short_kernel<<<dim3((unsigned)rows), dim3(256), 0, ctx->stream>>>(out, x, gamma, beta, residual, cols, eps);
    else rmsnorm_kernel<<<dim3((unsigned)rows), dim3(256), 0, ctx->stream>>>(out, x, gamma, beta, residual, cols, eps);
    LAUNCH_CHECK(ctx, "rmsnorm");
    return AIONHIP_OK;
}
int launch_gate_gelu(aionhip_ctx *ctx, float *out, const float *a, const float *b, size_t n) {
    gate_gelu_kernel<<<dim3(grid_for(n, 256)), dim3(256), 0, ctx->stream>>>(out, a, b, n);
    LAUNCH_CHECK(ctx, "gate_gelu");
    return AIONHIP_OK;
}

extern "C" {

int aionhip_step_rmsnorm(aionhip_ctx *ctx, aionhip_handle out, aionhip_handle x, aionhip_handle gamma, aionhip_handle beta,
                         aionhip_handle residual, size_t rows, size_t cols, float eps) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!out || !x || !gamma) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "rmsnorm: null operand");
    if (!(eps > 0.f) || !(eps < INFINITY)) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "rmsnorm: eps must be positive and finite");
    if (!rows || !cols) return AIONHIP_OK;
    if (rows > 0x7FFFFFFFu) return set_err(ctx, AIONHIP_UNSUPPORTED, "rmsnorm: too many rows");
    return launch_rmsnorm(ctx, dp<float>(out), dp<const float>(x), dp<const float>(gamma), dp<const float>(beta), dp<const float>(residual), rows, cols, eps);
}

int aionhip_step_rope(aionhip_ctx *ctx, aionhip_handle out, aionhip_handle x, aionhip_handle positions, size_t b, size_t t, size_t h,
                      size_t d, float base_frequency, float scale_factor, float rope_proportion) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!out || !x || !positions) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "rope: null operand");
    if (!(base_frequency > 0.f) || !(base_frequency < INFINITY) || !(scale_factor > 0.f) || !(scale_factor < INFINITY) ||
        !(rope_proportion >= 0.f && rope_proportion <= 1.f))
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "rope: base/scale must be positive and finite, proportion in [0,1]");
    if (d % 2 != 0 || d > 65534 || h > 65535) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "rope: head size must be even");
    const size_t tokens = b * t;
    if (!tokens || !h || !d) return AIONHIP_OK;
    const size_t half = d / 2;
    size_t rope_pairs = (size_t)floorf(rope_proportion * (float)half);
    if (rope_pairs > half) rope_pairs = half;
    const float freq_step = (float)pow((double)base_frequency, (double)(-2.0f / (float)d));
    const float *freq = nullptr;
    int rc = rope_table(ctx, (int)rope_pairs, freq_step, scale_factor, &freq);
    if (rc) return rc;
    rope_kernel<<<dim3(grid_for(tokens * half, 128)), dim3(128), 0, ctx->stream>>>(dp<float>(out), dp<const float>(x), dp<const int>(positions),
                                                                                   tokens, (int)h, (int)d, (int)rope_pairs, freq);
    LAUNCH_CHECK(ctx, "rope");
    return AIONHIP_OK;
}

int aionhip_step_rope_append(aionhip_ctx *ctx, aionhip_handle q_out, aionhip_handle q, aionhip_handle k, aionhip_handle v,
                             aionhip_handle k_cache, aionhip_handle v_cache, aionhip_handle positions, aionhip_handle write_index,
                             size_t b, size_t s, size_t t_cap, size_t h_q, size_t h_kv, size_t d, float base_frequency,
                             float scale_factor, float rope_proportion) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!q_out || !q || !k || !v || !k_cache || !v_cache || !positions || !write_index) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "rope_append: null operand");
    if (!(base_frequency > 0.f) || !(base_frequency < INFINITY) || !(scale_factor > 0.f) || !(scale_factor < INFINITY) ||
        !(rope_proportion >= 0.f && rope_proportion <= 1.f))
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "rope_append: base/scale must be positive and finite, proportion in [0,1]");
    if (d % 2 != 0 || d > 65534 || h_q > 65535 || h_kv > 65535) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "rope_append: head size must be even");
    if (s > t_cap) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "rope_append: %zu new tokens exceed the cache capacity %zu", s, t_cap);
    const size_t half = d / 2, total = b * s * half * (h_q + h_kv);
    if (!total || !h_q || !h_kv) return AIONHIP_OK;
    size_t rope_pairs = (size_t)floorf(rope_proportion * (float)half);
    if (rope_pairs > half) rope_pairs = half;
    const float freq_step = (float)pow((double)base_frequency, (double)(-2.0f / (float)d));
    const float *freq = nullptr;
    int rc = rope_table(ctx, (int)rope_pairs, freq_step, scale_factor, &freq);
    if (rc) return rc;
    rope_append_kernel<<<dim3(grid_for(total, 128)), dim3(128), 0, ctx->stream>>>(
        dp<float>(q_out), dp<const float>(q), dp<const float>(k), dp<const float>(v), dp<__half>(k_cache), dp<__half>(v_cache),
        dp<const int>(positions), dp<const int>(write_index), b, s, t_cap, (int)h_q, (int)h_kv, (int)d, (int)rope_pairs, freq);
    LAUNCH_CHECK(ctx, "rope_append");
    return AIONHIP_OK;
}

int aionhip_step_headnorm_rope_append(aionhip_ctx *ctx, aionhip_handle q_out, aionhip_handle q, aionhip_handle k, aionhip_handle v,
                                      aionhip_handle gamma_q, aionhip_handle beta_q, aionhip_handle gamma_k, aionhip_handle beta_k,
                                      aionhip_handle gamma_v, aionhip_handle beta_v, float eps, aionhip_handle k_cache,
                                      aionhip_handle v_cache, aionhip_handle positions, aionhip_handle write_index, size_t b, size_t s,
                                      size_t t_cap, size_t h_q, size_t h_kv, size_t d, float base_frequency, float scale_factor,
                                      float rope_proportion, int rolling) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!q_out || !q || !k || !v || !gamma_q || !gamma_k || !gamma_v || !k_cache || !v_cache || !positions || !write_index)
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "headnorm_rope_append: null operand");
    if (!(eps > 0.f) || !(eps < INFINITY)) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "headnorm_rope_append: eps must be positive and finite");
    if (!(base_frequency > 0.f) || !(base_frequency < INFINITY) || !(scale_factor > 0.f) || !(scale_factor < INFINITY) ||
        !(rope_proportion >= 0.f && rope_proportion <= 1.f))
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "headnorm_rope_append: base/scale must be positive and finite, proportion in [0,1]");
    if (d % 2 != 0 || h_q > 65535 || h_kv > 65535) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "headnorm_rope_append: head size must be even");
    if (d > 512) return set_err(ctx, AIONHIP_UNSUPPORTED, "headnorm_rope_append: head size %zu above 512 (issue the separate steps)", d);
    if (s > t_cap) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "headnorm_rope_append: %zu new tokens exceed the cache capacity %zu", s, t_cap);
    const size_t items = b * s * (h_q + 2 * h_kv);
    if (!items || !h_q || !h_kv || !d) return AIONHIP_OK;
    const size_t half = d / 2;
    size_t rope_pairs = (size_t)floorf(rope_proportion * (float)half);
    if (rope_pairs > half) rope_pairs = half;
    const float freq_step = (float)pow((double)base_frequency, (double)(-2.0f / (float)d));
    const float *freq = nullptr;
    int rc = rope_table(ctx, (int)rope_pairs, freq_step, scale_factor, &freq);
    if (rc) return rc;
    headnorm_rope_append_kernel<<<dim3(grid_for(items, 4)), dim3(256), 0, ctx->stream>>>(
        dp<float>(q_out), dp<const float>(q), dp<const float>(k), dp<const float>(v), dp<const float>(gamma_q), dp<const float>(beta_q),
        dp<const float>(gamma_k), dp<const float>(beta_k), dp<const float>(gamma_v), dp<const float>(beta_v), eps, dp<__half>(k_cache),
        dp<__half>(v_cache), dp<const int>(positions), dp<const int>(write_index), b, s, t_cap, (int)h_q, (int)h_kv, (int)d,
        (int)rope_pairs, freq, rolling);
    LAUNCH_CHECK(ctx, "headnorm_rope_append");
    return AIONHIP_OK;
}

int aionhip_step_add(aionhip_ctx *ctx, aionhip_handle out, aionhip_handle a, aionhip_handle b, size_t n) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!out || !a || !b) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "add: null operand");
    if (!n) return AIONHIP_OK;
    add_kernel<<<dim3(grid_for(n, 256)), dim3(256), 0, ctx->stream>>>(dp<float>(out), dp<const float>(a), dp<const float>(b), n);
    LAUNCH_CHECK(ctx, "add");
    return AIONHIP_OK;
}

int aionhip_step_unary(aionhip_ctx *ctx, int op, aionhip_handle out, aionhip_handle x, size_t n) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!out || !x) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "unary: null operand");
    if (op == 6) return set_err(ctx, AIONHIP_UNSUPPORTED, "unary: log has no step on this backend");
    if (op < 0 || op > 6) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "unary: unknown op %d", op);
    if (!n) return AIONHIP_OK;
    const dim3 grid(grid_for(n, 256)), block(256);
    float *o = dp<float>(out);
    const float *p = dp<const float>(x);
    switch (op) {
    case AIONHIP_UNARY_RELU: unary_kernel<AIONHIP_UNARY_RELU><<<grid, block, 0, ctx->stream>>>(o, p, n); break;
    case AIONHIP_UNARY_GELU: unary_kernel<AIONHIP_UNARY_GELU><<<grid, block, 0, ctx->stream>>>(o, p, n); break;
    case AIONHIP_UNARY_SILU: unary_kernel<AIONHIP_UNARY_SILU><<<grid, block, 0, ctx->stream>>>(o, p, n); break;
    case AIONHIP_UNARY_SIGMOID: unary_kernel<AIONHIP_UNARY_SIGMOID><<<grid, block, 0, ctx->stream>>>(o, p, n); break;
    case AIONHIP_UNARY_TANH: unary_kernel<AIONHIP_UNARY_TANH><<<grid, block, 0, ctx->stream>>>(o, p, n); break;
    default: unary_kernel<AIONHIP_UNARY_SQRT><<<grid, block, 0, ctx->stream>>>(o, p, n); break;
    }
    LAUNCH_CHECK(ctx, "unary");
    return AIONHIP_OK;
}

int aionhip_step_binary(aionhip_ctx *ctx, int op, aionhip_handle out, aionhip_handle a, aionhip_handle b, size_t n, size_t nb) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!out || !a || !b) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "binary: null operand");
    if (op < AIONHIP_BINARY_ADD || op > AIONHIP_BINARY_DIV) return set_err(ctx, AIONHIP_UNSUPPORTED, "binary: op %d has no step on this backend (add, sub, mul, div do)", op);
    if (!n) return AIONHIP_OK;
    if (nb == 0 || n % nb != 0) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "binary: b's %zu elements do not tile a's %zu", nb, n);
    const dim3 grid(grid_for(n, 256)), block(256);
    float *o = dp<float>(out);
    const float *pa = dp<const float>(a), *pb = dp<const float>(b);
    switch (op) {
    case AIONHIP_BINARY_ADD: binary_kernel<AIONHIP_BINARY_ADD><<<grid, block, 0, ctx->stream>>>(o, pa, pb, n, nb); break;
    case AIONHIP_BINARY_SUB: binary_kernel<AIONHIP_BINARY_SUB><<<grid, block, 0, ctx->stream>>>(o, pa, pb, n, nb); break;
    case AIONHIP_BINARY_MUL: binary_kernel<AIONHIP_BINARY_MUL><<<grid, block, 0, ctx->stream>>>(o, pa, pb, n, nb); break;
    default: binary_kernel<AIONHIP_BINARY_DIV><<<grid, block, 0, ctx->stream>>>(o, pa, pb, n, nb); break;
    }
    LAUNCH_CHECK(ctx, "binary");
    return AIONHIP_OK;
}

int aionhip_step_gate_gelu(aionhip_ctx *ctx, aionhip_handle out, aionhip_handle a, aionhip_handle b, size_t n) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!out || !a || !b) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "gate: null operand");
    if (!n) return AIONHIP_OK;
    return launch_gate_gelu(ctx, dp<float>(out), dp<const float>(a), dp<const float>(b), n);
}

int aionhip_step_gather_rows(aionhip_ctx *ctx, int table_dtype, aionhip_handle out, aionhip_handle table, aionhip_handle ids,
                             size_t n_ids, size_t d, size_t vocab) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (table_dtype != AIONHIP_F32 && table_dtype != AIONHIP_Q8_0) return set_err(ctx, AIONHIP_UNSUPPORTED, "gather: table must be f32 or q8_0");
    if (!out || !table || !ids) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "gather: null operand");
    if (table_dtype == AIONHIP_Q8_0 && d % QK != 0) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "gather: q8_0 row length must be a multiple of 32");
    if (!n_ids || !d) return AIONHIP_OK;
    if (n_ids > 0x7FFFFFFFu) return set_err(ctx, AIONHIP_UNSUPPORTED, "gather: too many ids");
    gather_rows_kernel<<<dim3((unsigned)n_ids), dim3(256), 0, ctx->stream>>>(table_dtype, dp<float>(out), dp<const void>(table), dp<const int>(ids), d, vocab);
    LAUNCH_CHECK(ctx, "gather_rows");
    return AIONHIP_OK;
}

int aionhip_step_append_f16(aionhip_ctx *ctx, aionhip_handle cache, aionhip_handle src_f32, aionhip_handle write_index, size_t b,
                            size_t s, size_t t_cap, size_t row_elems, int rolling) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!cache || !src_f32 || !write_index) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "append: null operand");
    if (s > t_cap) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "append: %zu new tokens exceed the cache capacity %zu", s, t_cap);
    const size_t total = b * s * row_elems;
    if (!total) return AIONHIP_OK;
    append_f16_kernel<<<dim3(grid_for(total, 256)), dim3(256), 0, ctx->stream>>>(dp<__half>(cache), dp<const float>(src_f32), dp<const int>(write_index),
                                                                                 s, t_cap, row_elems, total, rolling);
    LAUNCH_CHECK(ctx, "append_f16");
    return AIONHIP_OK;
}

int aionhip_step_sequence_append(aionhip_ctx *ctx, int dtype, aionhip_handle cache, aionhip_handle new_kv, aionhip_handle end_index, size_t b,
                                 size_t s, size_t t_cap, size_t row_elems, int rolling) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!cache || !new_kv || !end_index) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "sequence_append: null operand");
    if (dtype != AIONHIP_F16 && dtype != AIONHIP_F32) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "sequence_append: caches hold f16 or f32, not dtype %d", dtype);
    if (s > t_cap) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "sequence_append: %zu new tokens exceed the cache capacity %zu", s, t_cap);
    const size_t total = b * s * row_elems;
    if (!total) return AIONHIP_OK;
    if (dtype == AIONHIP_F16)
        append_same_kernel<unsigned short><<<dim3(grid_for(total, 256)), dim3(256), 0, ctx->stream>>>(
            dp<unsigned short>(cache), dp<const unsigned short>(new_kv), dp<const int>(end_index), s, t_cap, row_elems, total, rolling);
    else
        append_same_kernel<unsigned><<<dim3(grid_for(total, 256)), dim3(256), 0, ctx->stream>>>(
            dp<unsigned>(cache), dp<const unsigned>(new_kv), dp<const int>(end_index), s, t_cap, row_elems, total, rolling);
    LAUNCH_CHECK(ctx, "sequence_append");
    return AIONHIP_OK;
}

size_t aionhip_cache_grow_target(size_t current, size_t num, size_t den) {
    if (!current || !num || !den) return 0;
    if (current > SIZE_MAX / num) return 0;
    const size_t prod = current * num;
    if (prod > SIZE_MAX - (den - 1)) return 0;
    const size_t next = (prod + den - 1) / den;
    if (next <= current) return current == SIZE_MAX ? 0 : current + 1;
    return next;
}

int aionhip_cache_grow(aionhip_ctx *ctx, aionhip_handle dst, aionhip_handle src, size_t outer, size_t old_run_bytes, size_t new_run_bytes) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!dst || !src) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "cache_grow: null operand");
    if (dst == src) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "cache_grow: the grown cache needs a backing of its own");
    if ((old_run_bytes | new_run_bytes) & 3) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "cache_grow: runs of %zu and %zu bytes are not whole 4-byte words", old_run_bytes, new_run_bytes);
    if (new_run_bytes < old_run_bytes) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "cache_grow: %zu -> %zu bytes per run is not a growth", old_run_bytes, new_run_bytes);
    if (new_run_bytes && outer > SIZE_MAX / new_run_bytes) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "cache_grow: size overflow");
    const size_t total = outer * (new_run_bytes / 4);
    if (!total) return AIONHIP_OK;
    cache_grow_kernel<<<dim3(grid_for(total, 256)), dim3(256), 0, ctx->stream>>>(dp<unsigned>(dst), dp<const unsigned>(src), old_run_bytes / 4, new_run_bytes / 4, total);
    LAUNCH_CHECK(ctx, "cache_grow");
    return AIONHIP_OK;
}

int aionhip_cache_grow_rolling(aionhip_ctx *ctx, aionhip_handle dst, aionhip_handle src, aionhip_handle logical_ends, size_t b,
                               size_t old_capacity, size_t new_capacity, size_t row_bytes, size_t retained_history) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!dst || !src || !logical_ends) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "cache_grow_rolling: null operand");
    if (dst == src) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "cache_grow_rolling: the grown cache needs a backing of its own");
    if (!old_capacity || new_capacity <= old_capacity)
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "cache_grow_rolling: capacity %zu -> %zu is not a growth", old_capacity, new_capacity);
    if (row_bytes & 3) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "cache_grow_rolling: rows of %zu bytes are not whole 4-byte words", row_bytes);
    if (row_bytes && (new_capacity > SIZE_MAX / row_bytes || (b && new_capacity * row_bytes > SIZE_MAX / b)))
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "cache_grow_rolling: size overflow");
    const size_t total = b * new_capacity * (row_bytes / 4);
    if (!total) return AIONHIP_OK;
    cache_grow_rolling_kernel<<<dim3(grid_for(total, 256)), dim3(256), 0, ctx->stream>>>(dp<unsigned>(dst), dp<const unsigned>(src), dp<const int>(logical_ends),
                                                                                         old_capacity, new_capacity, row_bytes / 4, retained_history, total);
    LAUNCH_CHECK(ctx, "cache_grow_rolling");
    return AIONHIP_OK;
}

int aionhip_step_cast_f32_f16(aionhip_ctx *ctx, aionhip_handle out_f16, aionhip_handle x_f32, size_t n) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!out_f16 || !x_f32) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "cast: null operand");
    if (!n) return AIONHIP_OK;
    cast_f16_kernel<<<dim3(grid_for(n, 256)), dim3(256), 0, ctx->stream>>>(dp<__half>(out_f16), dp<const float>(x_f32), n);
    LAUNCH_CHECK(ctx, "cast_f32_f16");
    return AIONHIP_OK;
}

// Measurement aid: nothing but 16-byte non-temporal loads over `bytes` of `src`, 4 in flight per lane,
// the loaded words folded into a value that is stored only if it hits one unlikely constant. What this
// kernel reaches on a byte count is the device's practical read rate for that count (launch and ramp
// included); the GEMV kernels are reported beside it.
// Shape of the read: the one the one-row GEMV streams with - every wavefront takes one contiguous 4 KiB piece (four 16-byte
// loads per lane, each a contiguous KiB per wavefront, all four in flight at once) and ends; 512-thread workgroups, as many as
// there are pieces. (A persistent grid-stride loop with the same loads in flight reaches 5.7 TB/s on 300 MB where this reaches
// what the GEMV does.)
__global__ __launch_bounds__(512) void stream_read_kernel(const u32x4 *__restrict__ p, size_t n16, unsigned *sink) {
    const size_t piece = (size_t)blockIdx.x * 8 + (threadIdx.x >> 6);        // 256 chunks of 16 bytes each
    const size_t i0 = piece * 256 + (threadIdx.x & 63);
    u32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const size_t i = i0 + u * 64;
        v[u] = __builtin_nontemporal_load(p + (i < n16 ? i : n16 - 1));      // unconditional, clamped: the tail re-reads the last chunk
    }
    unsigned acc = 0;
#pragma unroll
    for (int u = 0; u < 4; ++u) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    if (acc == 0x9E3779B9u) *sink = acc;
}

int aionhip_probe_stream_read(aionhip_ctx *ctx, aionhip_handle src, size_t offset, size_t bytes, aionhip_handle sink) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!src || !sink) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "stream_read: null operand");
    if ((offset | bytes) & 15) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "stream_read: offset and size must be multiples of 16");
    if (!bytes) return AIONHIP_OK;
    const size_t n16 = bytes / 16;
    const size_t grid = (n16 + 2047) / 2048;                      // eight 4 KiB pieces per workgroup
    if (grid > 0x7FFFFFFFu) return set_err(ctx, AIONHIP_UNSUPPORTED, "stream_read: more than 8 TiB");
    ProfScope scope(ctx, "stream_read");
    launch_k(ctx, stream_read_kernel, dim3((unsigned)grid), dim3(512), 0, (const u32x4 *)(dp<const unsigned char>(src) + offset), n16, dp<unsigned>(sink));
    LAUNCH_CHECK(ctx, "stream_read");
    return AIONHIP_OK;
}

int aionhip_step_argmax(aionhip_ctx *ctx, aionhip_handle out_i32, aionhip_handle x, size_t rows, size_t n) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (!out_i32 || !x) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "argmax: null operand");
    if (n == 0) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "argmax: empty axis");
    if (!rows) return AIONHIP_OK;
    if (rows > 0x7FFFFFFFu || n > 0x7FFFFFFFu) return set_err(ctx, AIONHIP_UNSUPPORTED, "argmax: dimension too large");
    if (rows > 65535) return set_err(ctx, AIONHIP_UNSUPPORTED, "argmax: more than 65535 rows");
    int rc = ensure_scratch2(ctx, rows * ARGMAX_PARTS * 8);
    if (rc) return rc;
    rc = grow_work_buffer(ctx, &ctx->tickets, &ctx->tickets_bytes, rows * sizeof(unsigned), true, "the argmax tickets");
    if (rc) return rc;
    argmax_kernel<<<dim3(ARGMAX_PARTS, (unsigned)rows), dim3(256), 0, ctx->stream>>>(dp<int>(out_i32), (unsigned long long *)ctx->scratch2, (unsigned *)ctx->tickets,
                                                                                     dp<const float>(x), n);
    LAUNCH_CHECK(ctx, "argmax");
    return AIONHIP_OK;
}

}  // extern "C"
