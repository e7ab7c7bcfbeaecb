// Block quantizers (host and device) and the int8 activation preparation kernel.
//
// q8_0 follows aion storage/quantize.zig:83-103 (packQ8Block: codes against the f16-ROUNDED
// scale, clamp [-128,127]); q4_0 follows cpu/test_cpu_kernels.zig:490-523 (codes against the
// unrounded f32 scale, clamp [-8,7], nibble = code+8, even element in the low nibble).
// Rounding is half away from zero (Zig @round), f32->f16 is round-to-nearest-even.
#include "common.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

namespace {

// ------------------------------------------------------------------------------ host side
inline uint16_t half_bits_host(float v) {
    _Float16 h = (_Float16)v;  // IEEE RNE
    uint16_t b;
    std::memcpy(&b, &h, 2);
    return b;
}
inline float half_to_float_host(uint16_t b) {
    _Float16 h;
    std::memcpy(&h, &b, 2);
    return (float)h;
}

void host_block_q8(const float *v, size_t stride, uint8_t *dst) {
    float amax = 0.f;
    for (int t = 0; t < QK; ++t) amax = std::fmax(amax, std::fabs(v[t * stride]));
    const uint16_t sb = half_bits_host(amax == 0.f ? 1.f : amax / 127.f);
    const float eff = half_to_float_host(sb);
    const float inv = (amax == 0.f || eff == 0.f) ? 0.f : 1.f / eff;
    dst[0] = (uint8_t)sb;
    dst[1] = (uint8_t)(sb >> 8);
    for (int t = 0; t < QK; ++t) {
        float r = std::round(v[t * stride] * inv);
        r = std::fmin(127.f, std::fmax(-128.f, r));
        dst[2 + t] = (uint8_t)(int8_t)(int)r;
    }
}

void host_block_q4(const float *v, size_t stride, uint8_t *dst) {
    float amax = 0.f;
    for (int t = 0; t < QK; ++t) amax = std::fmax(amax, std::fabs(v[t * stride]));
    const float scale = amax == 0.f ? 1.f : amax / 7.f;
    const uint16_t sb = half_bits_host(scale);
    dst[0] = (uint8_t)sb;
    dst[1] = (uint8_t)(sb >> 8);
    for (int i = 0; i < 16; ++i) {
        int lo = (int)std::fmin(7.f, std::fmax(-8.f, std::round(v[(2 * i) * stride] / scale))) + 8;
        int hi = (int)std::fmin(7.f, std::fmax(-8.f, std::round(v[(2 * i + 1) * stride] / scale))) + 8;
        dst[2 + i] = (uint8_t)(lo | (hi << 4));
    }
}

// ------------------------------------------------------------------------------ device side
__device__ __forceinline__ void store_u16(uint8_t *p, unsigned v) { *reinterpret_cast<uint16_t *>(p) = (uint16_t)v; }

// one thread per block; `stride` = distance between a block's elements
template <int DT>
__global__ void quantize_rank2_kernel(const float *__restrict__ src, uint8_t *__restrict__ dst, size_t rows, size_t cols, int axis) {
    const size_t nblocks = rows * cols / QK;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nblocks) return;
    size_t base, stride;
    if (axis == 1) {
        const size_t bpr = cols / QK;
        base = (i / bpr) * cols + (i % bpr) * QK;
        stride = 1;
    } else {
        base = (i / cols) * QK * cols + (i % cols);
        stride = cols;
    }
    float v[QK];
    float amax = 0.f;
#pragma unroll
    for (int t = 0; t < QK; ++t) {
        v[t] = src[base + t * stride];
        amax = fmaxf(amax, fabsf(v[t]));
    }
    if (DT == AIONHIP_Q8_0) {
        uint8_t *o = dst + i * Q8_BYTES;
        const __half sh = __float2half_rn(amax == 0.f ? 1.f : amax / 127.f);
        const float eff = __half2float(sh);
        const float inv = (amax == 0.f || eff == 0.f) ? 0.f : 1.f / eff;
        store_u16(o, __half_as_ushort(sh));
#pragma unroll
        for (int t = 0; t < QK; t += 2) {
            const int q0 = (int)fminf(127.f, fmaxf(-128.f, roundf(v[t] * inv)));
            const int q1 = (int)fminf(127.f, fmaxf(-128.f, roundf(v[t + 1] * inv)));
            store_u16(o + 2 + t, (unsigned)(q0 & 0xFF) | ((unsigned)(q1 & 0xFF) << 8));
        }
    } else {
        uint8_t *o = dst + i * Q4_BYTES;
        const float scale = amax == 0.f ? 1.f : amax / 7.f;
        store_u16(o, __half_as_ushort(__float2half_rn(scale)));
#pragma unroll
        for (int t = 0; t < QK; t += 4) {
            unsigned w = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int q = (int)fminf(7.f, fmaxf(-8.f, roundf(v[t + j] / scale))) + 8;
                w |= (unsigned)q << (4 * j);
            }
            store_u16(o + 2 + t / 2, w);
        }
    }
}

// Activation preparation (aion matmul_q_i8.zig:187-203): 8 lanes share one 32-element block.
// GATE: the activation is gelu_tanh(a) * up (aion cpu/exec/elementwise.zig:25-37), not written out.
// RMSNorm + int8 preparation, one workgroup per row of k columns (k a multiple of 32; x, gamma, beta 16-byte aligned). The sum
// of squares runs in the norm kernels' order (thread c of 256 adds x[c]^2, x[c + 256]^2, ...; then block_sum_256) and a value
// is rounded as they round it ((x * inv) * gamma + beta), so the codes, scales and code sums are those of the norm step followed
// by the preparation launch. SHORT: rows of up to 2048 columns, every load requested before the reduction (one memory round
// trip); otherwise two passes over the row.
template <bool SHORT>
__global__ __launch_bounds__(256) void rmsnorm_prepare_kernel(const float *__restrict__ x, const float *__restrict__ gamma, const float *__restrict__ beta,
                                                              size_t cols, float eps, int *__restrict__ aq, float *__restrict__ a_scale,
                                                              int *__restrict__ a_sum) {
    __shared__ float red[4];
    const size_t row = blockIdx.x;
    const float *xr = x + row * cols;
    const size_t chunks = cols >> 2, kb_per_row = cols / QK;
    const int tid = threadIdx.x;
    auto emit = [&](size_t c4, bool live, f32x4 xv, f32x4 gv, f32x4 bv, float inv) {
        const float y0 = (xv.x * inv) * gv.x + (beta ? bv.x : 0.f), y1 = (xv.y * inv) * gv.y + (beta ? bv.y : 0.f);
        const float y2 = (xv.z * inv) * gv.z + (beta ? bv.z : 0.f), y3 = (xv.w * inv) * gv.w + (beta ? bv.w : 0.f);
        int word, sm;
        float scale;
        prepare_act_block8(y0, y1, y2, y3, word, scale, sm);         // (all eight lanes of a block take part: chunks is a multiple of 8)
        if (live) {
            aq[row * chunks + c4] = word;
            if ((c4 & 7) == 0) {
                a_scale[row * kb_per_row + (c4 >> 3)] = scale;
                a_sum[row * kb_per_row + (c4 >> 3)] = sm;
            }
        }
    };
    const f32x4 *x4 = (const f32x4 *)xr, *g4 = (const f32x4 *)gamma, *b4 = (const f32x4 *)(beta ? beta : gamma);
    if (SHORT) {
        float sv[8];
        f32x4 xc[2], gc[2], bc[2];
#pragma unroll
        for (int j = 0; j < 8; ++j) sv[j] = xr[min((size_t)tid + 256 * j, cols - 1)];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const size_t c4 = min((size_t)tid + 256 * i, chunks - 1);
            xc[i] = x4[c4];
            gc[i] = g4[c4];
            bc[i] = b4[c4];
        }
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if ((size_t)tid + 256 * j < cols) ss += sv[j] * sv[j];
        ss = block_sum_256(ss, red);
        const float inv = 1.f / sqrtf(ss * (1.f / (float)cols) + eps);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const size_t c4 = (size_t)tid + 256 * i;
            if (256 * (size_t)i < chunks) emit(c4, c4 < chunks, xc[i], gc[i], bc[i], inv);      // (uniform per workgroup)
        }
    } else {
        float ss = 0.f;
        for (size_t c = tid; c < cols; c += 256) ss += xr[c] * xr[c];
        ss = block_sum_256(ss, red);
        const float inv = 1.f / sqrtf(ss * (1.f / (float)cols) + eps);
        for (size_t base = 0; base < chunks; base += 256) {
            const size_t c4 = base + tid, cc = min(c4, chunks - 1);
            emit(c4, c4 < chunks, x4[cc], g4[cc], b4[cc], inv);
        }
    }
}

template <bool GATE>
__global__ __launch_bounds__(256) void prepare_act_kernel(const float *__restrict__ a, const float *__restrict__ up, size_t lda, size_t m, size_t k,
                                                          int *__restrict__ aq, float *__restrict__ a_scale, int *__restrict__ a_sum) {
    const size_t kb_per_row = k / QK;
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t blk = gid >> 3;
    const int sub = (int)(gid & 7);
    const bool live = blk < m * kb_per_row;
    const size_t row = live ? blk / kb_per_row : 0, kb = live ? blk % kb_per_row : 0;
    const float *p = a + row * lda + kb * QK + sub * 4;
    float v0 = 0.f, v1 = 0.f, v2 = 0.f, v3 = 0.f;
    if (live) { v0 = p[0]; v1 = p[1]; v2 = p[2]; v3 = p[3]; }
    if (GATE && live) {
        const float *u = up + row * lda + kb * QK + sub * 4;
        v0 = aion_gate_gelu(v0, u[0]);
        v1 = aion_gate_gelu(v1, u[1]);
        v2 = aion_gate_gelu(v2, u[2]);
        v3 = aion_gate_gelu(v3, u[3]);
    }
    int word, s;
    float scale;
    prepare_act_block8(v0, v1, v2, v3, word, scale, s);
    if (live) {
        aq[(row * k + kb * QK) / 4 + sub] = word;
        if (sub == 0) {
            a_scale[row * kb_per_row + kb] = scale;
            a_sum[row * kb_per_row + kb] = s;
        }
    }
}

}  // namespace

size_t prepared_act_bytes(size_t m, size_t k) {
    const size_t q = (m * k + 255) & ~(size_t)255;
    const size_t s = (m * (k / QK) * 4 + 255) & ~(size_t)255;
    return q + 2 * s;
}
PreparedAct prepared_act_carve(void *base, size_t m, size_t k) {
    const size_t q = (m * k + 255) & ~(size_t)255;
    const size_t s = (m * (k / QK) * 4 + 255) & ~(size_t)255;
    PreparedAct p;
    p.q = (int8_t *)base;
    p.scale = (float *)((char *)base + q);
    p.sum = (int *)((char *)base + q + s);
    return p;
}
int launch_prepare_act(aionhip_ctx *ctx, const float *a, size_t lda, size_t m, size_t k, PreparedAct out) {
    const size_t threads = m * (k / QK) * 8;
    if (!threads) return AIONHIP_OK;
    const size_t blocks = (threads + 255) / 256;
    ProfScope scope(ctx, "prepare_act");
    launch_k(ctx, prepare_act_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, a, nullptr, lda, m, k, (int *)out.q, out.scale, out.sum);
    LAUNCH_CHECK(ctx, "prepare_act");
    return AIONHIP_OK;
}
int launch_prepare_gate(aionhip_ctx *ctx, const float *gate, const float *up, size_t m, size_t k, PreparedAct out) {
    const size_t threads = m * (k / QK) * 8;
    if (!threads) return AIONHIP_OK;
    const size_t blocks = (threads + 255) / 256;
    ProfScope scope(ctx, "prepare_gate");
    launch_k(ctx, prepare_act_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, gate, up, k, m, k, (int *)out.q, out.scale, out.sum);
    LAUNCH_CHECK(ctx, "prepare_gate");
    return AIONHIP_OK;
}

// StepRMSNorm (cpu/exec/layernorm.zig:54-155) followed by the int8 preparation of its rows, as one launch: what the norm step
// and the preparation launch give, to the bit, without the normalized rows' trip through memory.
int launch_prepare_rmsnorm(aionhip_ctx *ctx, const float *x, const float *gamma, const float *beta, float eps, size_t m, size_t k, PreparedAct out) {
    if (!m || !k) return AIONHIP_OK;
    ProfScope scope(ctx, "prepare_rmsnorm");
    if (k <= 2048) launch_k(ctx, rmsnorm_prepare_kernel<true>, dim3((unsigned)m), dim3(256), 0, x, gamma, beta, k, eps, (int *)out.q, out.scale, out.sum);
    else launch_k(ctx, rmsnorm_prepare_kernel<false>, dim3((unsigned)m), dim3(256), 0, x, gamma, beta, k, eps, (int *)out.q, out.scale, out.sum);
    LAUNCH_CHECK(ctx, "prepare_rmsnorm");
    return AIONHIP_OK;
}

extern "C" {

int aionhip_quantize_blocks(int dtype, const size_t *shape, size_t rank, size_t quant_axis, const float *values, size_t n_values,
                            size_t first_elem, size_t first_block, uint8_t *out, size_t out_len) {
    if (dtype != AIONHIP_Q8_0 && dtype != AIONHIP_Q4_0) return AIONHIP_UNSUPPORTED;
    if (!shape || rank == 0 || rank > 8 || quant_axis >= rank || !out || !values) return AIONHIP_INVALID_ARGUMENT;
    const size_t bb = dtype == AIONHIP_Q8_0 ? Q8_BYTES : Q4_BYTES;
    if (shape[quant_axis] % QK != 0 || out_len % bb != 0) return AIONHIP_INVALID_ARGUMENT;
    size_t strides[8], bshape[8], total = 1;
    for (size_t d = rank; d-- > 0;) {
        strides[d] = total;
        if (shape[d] != 0 && total > SIZE_MAX / shape[d]) return AIONHIP_INVALID_ARGUMENT;
        total *= shape[d];
        bshape[d] = d == quant_axis ? shape[d] / QK : shape[d];
    }
    // Block-space index i = (outer * KB + kb) * inner + j, where `inner` is the product of the
    // dims after the quant axis (the distance between a block's elements) and KB the blocks along
    // the axis; its first element sits at outer*axis_len*inner + kb*32*inner + j.
    const size_t inner = strides[quant_axis];
    const size_t KB = bshape[quant_axis];
    const size_t axis_len = shape[quant_axis];
    const size_t total_blocks = total / QK;
    const size_t nb = out_len / bb;
    if (first_block > total_blocks || nb > total_blocks - first_block) return AIONHIP_INVALID_ARGUMENT;
    auto base_of = [&](size_t block) -> size_t {
        const size_t j = block % inner, kb = (block / inner) % KB, outer = block / (inner * KB);
        return outer * axis_len * inner + kb * QK * inner + j;
    };
    // validate the whole range first so that a failing call writes nothing (bases grow with the
    // block index inside one (outer, kb) run and across runs, so the ends bound the range)
    if (nb) {
        const size_t lo = base_of(first_block), hi = base_of(first_block + nb - 1) + (QK - 1) * inner;
        if (lo < first_elem || hi - first_elem >= n_values) return AIONHIP_INVALID_ARGUMENT;
    }
    unsigned hw = std::thread::hardware_concurrency();
    size_t nthreads = std::min<size_t>(hw ? hw : 1, 16);
    if (nb < 4096) nthreads = 1;
    auto work = [&](size_t lo, size_t hi) {
        constexpr size_t TILE = 64;
        float buf[TILE * QK];
        size_t i = lo;
        while (i < hi) {
            const size_t blk = first_block + i;
            const size_t local = base_of(blk) - first_elem;
            if (inner == 1) {
                if (dtype == AIONHIP_Q8_0) host_block_q8(values + local, 1, out + i * bb);
                else host_block_q4(values + local, 1, out + i * bb);
                ++i;
                continue;
            }
            // a run of blocks whose elements interleave in memory: gather 32 rows of `run` floats
            const size_t run = std::min(std::min(TILE, hi - i), inner - blk % inner);
            for (int t = 0; t < QK; ++t) {
                const float *src = values + local + (size_t)t * inner;
                for (size_t j = 0; j < run; ++j) buf[j * QK + t] = src[j];
            }
            for (size_t j = 0; j < run; ++j) {
                if (dtype == AIONHIP_Q8_0) host_block_q8(buf + j * QK, 1, out + (i + j) * bb);
                else host_block_q4(buf + j * QK, 1, out + (i + j) * bb);
            }
            i += run;
        }
    };
    if (nthreads <= 1) {
        work(0, nb);
    } else {
        std::vector<std::thread> pool;
        const size_t per = (nb + nthreads - 1) / nthreads;
        for (size_t t = 0; t < nthreads; ++t) {
            const size_t lo = t * per, hi = std::min(nb, lo + per);
            if (lo < hi) pool.emplace_back(work, lo, hi);
        }
        for (auto &th : pool) th.join();
    }
    return AIONHIP_OK;
}

int aionhip_quantize_device(aionhip_ctx *ctx, int dtype, size_t rows, size_t cols, size_t quant_axis,
                            aionhip_handle src_f32, aionhip_handle dst_blocks) {
    if (!ctx) return AIONHIP_INVALID_ARGUMENT;
    if (dtype != AIONHIP_Q8_0 && dtype != AIONHIP_Q4_0) return set_err(ctx, AIONHIP_UNSUPPORTED, "quantize: dtype %d is not block-quantized", dtype);
    if (quant_axis > 1 || !src_f32 || !dst_blocks) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "quantize: bad axis or null buffer");
    if ((quant_axis == 0 ? rows : cols) % QK != 0) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "quantize: axis length is not a multiple of 32");
    const size_t nblocks = rows * cols / QK;
    if (!nblocks) return AIONHIP_OK;
    const unsigned grid = (unsigned)((nblocks + 127) / 128);
    const float *s = (const float *)(uintptr_t)src_f32;
    uint8_t *d = (uint8_t *)(uintptr_t)dst_blocks;
    if (dtype == AIONHIP_Q8_0) quantize_rank2_kernel<AIONHIP_Q8_0><<<dim3(grid), dim3(128), 0, ctx->stream>>>(s, d, rows, cols, (int)quant_axis);
    else quantize_rank2_kernel<AIONHIP_Q4_0><<<dim3(grid), dim3(128), 0, ctx->stream>>>(s, d, rows, cols, (int)quant_axis);
    LAUNCH_CHECK(ctx, "quantize_rank2");
    return AIONHIP_OK;
}

}  // extern "C"
