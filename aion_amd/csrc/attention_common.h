// Shared by the attention kernels: argument block, element conversions, the interval window of a query, the row map of
// rolling caches (attention.hip, attention_prefill.hip).
#pragma once
#include "common.h"

#include <climits>
#include <type_traits>

namespace attn {


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

using u32x2 = __attribute__((ext_vector_type(2))) unsigned int;
// f(integral_constant<int, I>) for I in [I0, E): a loop whose index is a constant expression in the body (immediate
// operands of assembly, if constexpr)
template <int I, int E, class F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < E) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, E>(f);
    }
}

// ---- prefill kernel (attention_prefill.hip): 128 query rows per workgroup, 64-key tiles
constexpr int PF_ROWS = 128, PF_TK = 64;
#ifndef PF_FLASH_BELOW
#define PF_FLASH_BELOW 8   // prompts whose 128-row workgroups would fill under 1/PF_FLASH_BELOW of the CUs (head size 256; more at smaller heads) run on the 16-row split kernel
#endif
// whether the prefill kernel takes this call (head size 64, 128 or 256; K/V f16 or bf16; not the hi+lo precise mode)
bool prefill_takes(const AttnArgs &a, int d);
int launch_prefill(aionhip_ctx *ctx, AttnArgs &a, int d);

}  // namespace attn
