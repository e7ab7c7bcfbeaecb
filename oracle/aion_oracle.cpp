// CPU oracle for the aion quantized-inference hot path: TEST INFRASTRUCTURE ONLY.
// See aion_oracle.h for scope, pinning status and the reference citations; paths
// below are relative to the aion source tree (src/aion/...).
#include "aion_oracle.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <limits>
#include <map>
#include <string>
#include <thread>
#include <vector>

namespace {

constexpr size_t QK = 32;       // backend/types.zig:40-50: 32 elements per block
constexpr size_t Q8_BYTES = 34; // 2 B f16 scale + 32 x i8
constexpr size_t Q4_BYTES = 18; // 2 B f16 scale + 16 B nibbles

inline uint32_t f32_bits(float v) { uint32_t u; std::memcpy(&u, &v, 4); return u; }
inline float bits_f32(uint32_t u) { float v; std::memcpy(&v, &u, 4); return v; }

// IEEE binary32 -> binary16, round to nearest even, overflow -> inf, subnormals kept.
uint16_t f32_to_f16_bits(float v) {
    const uint32_t x = f32_bits(v);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t ax = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u) return (uint16_t)(sign | 0x7C00u | ((ax > 0x7F800000u) ? (0x0200u | ((ax >> 13) & 0x3FFu)) : 0u));
    if (ax >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);  // rounds to >= 65520 -> inf
    if (ax < 0x33000001u) return (uint16_t)sign;               // < 2^-25 (or exactly 2^-25 -> ties to even = 0)
    int32_t e = (int32_t)(ax >> 23) - 127;
    uint32_t man = (ax & 0x7FFFFFu) | 0x800000u;  // 24-bit significand
    int shift;                                      // bits to drop
    uint32_t base;
    if (e < -14) { shift = 13 + (-14 - e); base = 0; }      // subnormal half
    else { shift = 13; base = (uint32_t)(e + 15) << 10; man &= 0x7FFFFFu; }
    const uint32_t kept = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    uint32_t r = base + kept;
    if (rem > half || (rem == half && (kept & 1u))) r += 1;  // carry into the exponent is correct
    return (uint16_t)(sign | r);
}

float f16_bits_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1Fu;
    const uint32_t m = h & 0x3FFu;
    if (e == 0) {
        if (m == 0) return bits_f32(sign);
        float f = std::ldexp((float)m, -24);
        return sign ? -f : f;
    }
    if (e == 31) return bits_f32(sign | 0x7F800000u | (m << 13));
    return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}

void parallel_for(size_t n, int threads, const std::function<void(size_t, size_t)> &fn) {
    size_t t = threads < 1 ? 1 : (size_t)threads;
    if (t > n) t = n ? n : 1;
    if (t <= 1) { fn(0, n); return; }
    std::vector<std::thread> pool;
    const size_t per = (n + t - 1) / t;
    for (size_t i = 0; i < t; ++i) {
        const size_t lo = i * per, hi = std::min(n, lo + per);
        if (lo >= hi) break;
        pool.emplace_back([=, &fn] { fn(lo, hi); });
    }
    for (auto &th : pool) th.join();
}

// storage/quantize.zig:83-103
void pack_q8_block(const float *v, size_t stride, uint8_t *dst) {
    float absmax = 0.0f;
    for (size_t t = 0; t < QK; ++t) absmax = std::max(absmax, std::fabs(v[t * stride]));
    const float scale = absmax == 0.0f ? 1.0f : absmax / 127.0f;
    const uint16_t sbits = f32_to_f16_bits(scale);
    dst[0] = (uint8_t)(sbits & 0xFF);
    dst[1] = (uint8_t)(sbits >> 8);
    const float eff = f16_bits_to_f32(sbits);
    const float inv = (absmax == 0.0f || eff == 0.0f) ? 0.0f : 1.0f / eff;
    for (size_t t = 0; t < QK; ++t) {
        const float r = std::round(v[t * stride] * inv);  // half away from zero (Zig @round)
        int32_t q = r >= 2147483520.0f ? 2147483647 : (r <= -2147483648.0f ? INT32_MIN : (int32_t)r);
        q = std::max(-128, std::min(127, q));
        dst[2 + t] = (uint8_t)(int8_t)q;
    }
}

// cpu/test_cpu_kernels.zig:490-523 (divides by the UNROUNDED f32 scale)
void pack_q4_block(const float *v, size_t stride, uint8_t *dst) {
    float max_abs = 0.0f;
    for (size_t t = 0; t < QK; ++t) max_abs = std::max(max_abs, std::fabs(v[t * stride]));
    const float scale = max_abs == 0.0f ? 1.0f : max_abs / 7.0f;
    const uint16_t sbits = f32_to_f16_bits(scale);
    dst[0] = (uint8_t)(sbits & 0xFF);
    dst[1] = (uint8_t)(sbits >> 8);
    std::memset(dst + 2, 0, 16);
    for (size_t t = 0; t < QK; ++t) {
        const float qf = v[t * stride] / scale;
        int32_t q = (int32_t)std::round(qf);
        q = std::max(-8, std::min(7, q));
        const uint8_t nib = (uint8_t)(q + 8);
        if ((t & 1) == 0) dst[2 + (t >> 1)] = (uint8_t)((dst[2 + (t >> 1)] & 0xF0) | nib);
        else dst[2 + (t >> 1)] = (uint8_t)((dst[2 + (t >> 1)] & 0x0F) | (nib << 4));
    }
}

inline float block_scale(const uint8_t *blk) { return f16_bits_to_f32((uint16_t)(blk[0] | (blk[1] << 8))); }

// matmul_q_i8.zig:362-370: q4 code = nibble - 8; q8 code = i8
inline void block_codes(int dtype, const uint8_t *blk, int8_t *q) {
    if (dtype == ORC_Q8_0) {
        for (size_t t = 0; t < QK; ++t) q[t] = (int8_t)blk[2 + t];
    } else {
        for (size_t t = 0; t < QK; ++t) {
            const uint8_t b = blk[2 + (t >> 1)];
            q[t] = (int8_t)((int)((t & 1) ? (b >> 4) : (b & 15)) - 8);
        }
    }
}

// storage/quantize.zig:49-80: block-space traversal, row-major over `shape` with the quant
// axis divided by 32; a block's elements are `axis_stride` apart.
template <class F>
int for_each_block(const size_t *shape, size_t rank, size_t axis, F &&fn) {
    if (rank == 0 || rank > 8 || axis >= rank) return -1;
    if (shape[axis] % QK != 0) return -1;
    size_t strides[8], bshape[8];
    size_t s = 1;
    for (size_t d = rank; d-- > 0;) {
        strides[d] = s;
        s *= shape[d];
        bshape[d] = d == axis ? shape[d] / QK : shape[d];
    }
    size_t nblocks = 1;
    for (size_t d = 0; d < rank; ++d) nblocks *= bshape[d];
    for (size_t i = 0; i < nblocks; ++i) {
        size_t rest = i, base = 0;
        for (size_t d = rank; d-- > 0;) {
            const size_t c = rest % bshape[d];
            rest /= bshape[d];
            base += (d == axis ? c * QK : c) * strides[d];
        }
        fn(i, base, strides[axis]);
    }
    return 0;
}

// matmul_q_i8.zig:187-203
float quantize_a_block(const float *a, int8_t *out) {
    float amax = 0.0f;
    for (size_t t = 0; t < QK; ++t) amax = std::max(amax, std::fabs(a[t]));
    if (amax == 0.0f) { std::memset(out, 0, QK); return 0.0f; }
    const float scale = amax / 127.0f;
    const float inv = 127.0f / amax;
    for (size_t t = 0; t < QK; ++t) {
        float r = std::round(a[t] * inv);
        r = std::max(-127.0f, std::min(127.0f, r));
        out[t] = (int8_t)(int32_t)r;
    }
    return scale;
}

struct Prepared {
    std::vector<int8_t> q;
    std::vector<float> scale;
    size_t blocks = 0;
    void run(const float *a_row, size_t nb) {
        blocks = nb;
        q.resize(nb * QK);
        scale.resize(nb);
        for (size_t kb = 0; kb < nb; ++kb) scale[kb] = quantize_a_block(a_row + kb * QK, q.data() + kb * QK);
    }
};

// matmul_q_i8.zig:211-225 (dotI8Narrow on the 8-lane byte dot): lane j of the folded dot
// covers bytes [4j,4j+4) and [16+4j,16+4j+4).
inline void dot_narrow(const int8_t *a, const int8_t *b, int32_t d[4]) {
    for (int j = 0; j < 4; ++j) {
        int32_t s = 0;
        for (int t = 0; t < 4; ++t) s += (int32_t)a[4 * j + t] * b[4 * j + t] + (int32_t)a[16 + 4 * j + t] * b[16 + 4 * j + t];
        d[j] = s;
    }
}
inline float reduce4(const float l[4]) { return (l[0] + l[2]) + (l[1] + l[3]); }

inline float store_c(float alpha, float beta, float dot, float c_old) {
    return beta == 0.0f ? alpha * dot : alpha * dot + beta * c_old;
}

// ---- fast_math.zig:53-148 ----
inline float clampf(float x, float lo, float hi) { return std::max(lo, std::min(hi, x)); }
float exp_approx(float x_in) {
    const float x = clampf(x_in, -80.0f, 80.0f);
    const float inv_ln2 = 1.4426950408889634f, ln2 = 0.6931471805599453f;
    const float y = x * inv_ln2;
    const int32_t n = (int32_t)std::floor(y + 0.5f);
    const float r = y - (float)n;
    const float t = r * ln2;
    const float c4 = 1.0f / 24.0f, c3 = 1.0f / 6.0f, c2 = 0.5f;
    const float p = 1.0f + t * (1.0f + t * (c2 + t * (c3 + t * c4)));
    return bits_f32((uint32_t)(n + 127) << 23) * p;
}
float sigmoid_approx(float x) {
    float y;
    if (x >= 0.0f) { const float e = exp_approx(-x); y = 1.0f / (1.0f + e); }
    else { const float e = exp_approx(x); y = e / (1.0f + e); }
    return clampf(y, 0.0f, 1.0f);
}
float tanh_approx(float x) { return clampf(2.0f * sigmoid_approx(2.0f * x) - 1.0f, -1.0f, 1.0f); }
// kernels/attention.zig:42-48
float exp_softmax(float x) {
    if (!std::isfinite(x)) return x < 0.0f ? 0.0f : std::numeric_limits<float>::infinity();
    return exp_approx(clampf(x, -20.0f, 0.0f));
}

// graph/graph.zig:160-167
inline void window_keys(uint32_t left, uint32_t right, uint32_t chunk, size_t pos, size_t kv_end, size_t &lo, size_t &hi) {
    const size_t anchor = chunk > 0 ? (pos / chunk) * chunk : pos;
    const size_t span = chunk > 0 ? chunk : 1;
    lo = anchor - std::min(anchor, (size_t)left);
    size_t up = anchor + span;           // saturating adds in the reference; sizes here never overflow
    up = (right == 0xFFFFFFFFu) ? std::numeric_limits<size_t>::max() : up + (size_t)right;
    hi = std::min(kv_end, up);
}

inline float kv_at(const void *p, int dtype, size_t idx) {
    return dtype == 0 ? ((const float *)p)[idx] : f16_bits_to_f32(((const uint16_t *)p)[idx]);
}

}  // namespace

extern "C" {

uint16_t orc_f32_to_f16(float v) { return f32_to_f16_bits(v); }
float orc_f16_to_f32(uint16_t b) { return f16_bits_to_f32(b); }
float orc_exp_approx(float x) { return exp_approx(x); }
float orc_tanh_approx(float x) { return tanh_approx(x); }

int orc_quantize(int dtype, const size_t *shape, size_t rank, size_t axis, const float *values, uint8_t *out) {
    if (dtype != ORC_Q8_0 && dtype != ORC_Q4_0) return -1;
    const size_t bb = dtype == ORC_Q8_0 ? Q8_BYTES : Q4_BYTES;
    return for_each_block(shape, rank, axis, [&](size_t i, size_t base, size_t stride) {
        if (dtype == ORC_Q8_0) pack_q8_block(values + base, stride, out + i * bb);
        else pack_q4_block(values + base, stride, out + i * bb);
    });
}

int orc_dequantize(int dtype, const size_t *shape, size_t rank, size_t axis, const uint8_t *blocks, float *out) {
    if (dtype != ORC_Q8_0 && dtype != ORC_Q4_0) return -1;
    const size_t bb = dtype == ORC_Q8_0 ? Q8_BYTES : Q4_BYTES;
    return for_each_block(shape, rank, axis, [&](size_t i, size_t base, size_t stride) {
        int8_t q[QK];
        block_codes(dtype, blocks + i * bb, q);
        const float s = block_scale(blocks + i * bb);
        for (size_t t = 0; t < QK; ++t) out[base + t * stride] = (float)q[t] * s;
    });
}

void orc_prepare_a(const float *a, size_t m, size_t k, size_t lda, int8_t *aq, float *a_scale, int32_t *a_sum) {
    const size_t nb = k / QK;
    for (size_t r = 0; r < m; ++r)
        for (size_t kb = 0; kb < nb; ++kb) {
            int8_t *q = aq + r * k + kb * QK;
            a_scale[r * nb + kb] = quantize_a_block(a + r * lda + kb * QK, q);
            int32_t s = 0;
            for (size_t t = 0; t < QK; ++t) s += q[t];
            if (a_sum) a_sum[r * nb + kb] = s;
        }
}

int orc_matmul_nt_q8(size_t m, size_t n, size_t k, float alpha, float beta, const float *a, size_t lda,
                     const uint8_t *b, float *c, size_t ldc, int threads) {
    if (k % QK != 0) return -1;
    if (lda == 0) lda = k;
    if (ldc == 0) ldc = n;
    const size_t nb = k / QK;
    // matmul_nt_q.zig:538-543: A is quantized once per call, every column reads the same slots.
    std::vector<Prepared> prep(m);
    for (size_t r = 0; r < m; ++r) prep[r].run(a + r * lda, nb);
    parallel_for(n, threads, [&](size_t lo, size_t hi) {
        for (size_t j = lo; j < hi; ++j) {
            const uint8_t *col = b + j * nb * Q8_BYTES;
            for (size_t r = 0; r < m; ++r) {
                float lanes[4] = {0, 0, 0, 0};
                for (size_t kb = 0; kb < nb; ++kb) {
                    const uint8_t *bp = col + kb * Q8_BYTES;
                    int32_t d[4];
                    dot_narrow((const int8_t *)(bp + 2), prep[r].q.data() + kb * QK, d);
                    const float s = prep[r].scale[kb] * block_scale(bp);  // matmul_nt_q.zig:74-80
                    for (int l = 0; l < 4; ++l) lanes[l] += (float)d[l] * s;
                }
                float &dst = c[r * ldc + j];
                dst = store_c(alpha, beta, reduce4(lanes), dst);
            }
        }
    });
    return 0;
}

int orc_matmul_q8_kmajor(size_t m, size_t n, size_t k, float alpha, float beta, const float *a, size_t lda,
                         const uint8_t *b, size_t ldb, float *c, size_t ldc, int threads) {
    if (k % QK != 0) return -1;
    if (lda == 0) lda = k;
    if (ldb == 0) ldb = n;
    if (ldc == 0) ldc = n;
    const size_t blocks = k / QK;
    const size_t chunk_blocks = 8192 / QK;  // matvec_q.zig:27 DOT_MAX_K
    for (size_t r = 0; r < m; ++r) {
        for (size_t kb0 = 0; kb0 < blocks; kb0 += chunk_blocks) {
            const size_t nb = std::min(chunk_blocks, blocks - kb0);
            Prepared prep;
            prep.run(a + r * lda + kb0 * QK, nb);
            const bool first = kb0 == 0;
            parallel_for(n, threads, [&](size_t lo, size_t hi) {
                for (size_t j = lo; j < hi; ++j) {
                    float lanes[4] = {0, 0, 0, 0};
                    for (size_t kb = 0; kb < nb; ++kb) {
                        const uint8_t *bp = b + ((kb0 + kb) * ldb + j) * Q8_BYTES;
                        int32_t d[4];
                        dot_narrow((const int8_t *)(bp + 2), prep.q.data() + kb * QK, d);
                        const float s = prep.scale[kb] * block_scale(bp);  // matvec_q.zig:139
                        for (int l = 0; l < 4; ++l) lanes[l] += (float)d[l] * s;
                    }
                    float &dst = c[r * ldc + j];
                    const float dot = reduce4(lanes);
                    dst = first ? store_c(alpha, beta, dot, dst) : dst + alpha * dot;  // matvec_q.zig:118-122
                }
            });
        }
    }
    return 0;
}

int orc_matmul_q_packed(int dtype, size_t m, size_t n, size_t k, float alpha, float beta, const float *a, size_t lda,
                        const uint8_t *b, float *c, size_t ldc, size_t kc, int threads) {
    if (dtype != ORC_Q8_0 && dtype != ORC_Q4_0) return -1;
    if (k % QK != 0 || kc == 0 || kc % QK != 0) return -1;
    if (lda == 0) lda = k;
    if (ldc == 0) ldc = n;
    const size_t bb = dtype == ORC_Q8_0 ? Q8_BYTES : Q4_BYTES;
    const size_t nb = k / QK;
    std::vector<int8_t> aq(m * k);
    std::vector<float> as(m * nb);
    orc_prepare_a(a, m, k, lda, aq.data(), as.data(), nullptr);  // matmul_q_i8.zig:423-433
    parallel_for(n, threads, [&](size_t lo, size_t hi) {
        for (size_t j = lo; j < hi; ++j) {
            for (size_t r = 0; r < m; ++r) {
                // exec/matmul.zig:429-435: K walked in kc steps, beta = 1 after the first.
                for (size_t pc = 0; pc < k; pc += kc) {
                    const size_t kw = std::min(kc, k - pc);
                    float cacc = 0.0f;
                    for (size_t kb = pc / QK; kb < (pc + kw) / QK; ++kb) {
                        const uint8_t *bp = b + (kb * n + j) * bb;
                        int8_t wq[QK];
                        block_codes(dtype, bp, wq);
                        int32_t idot = 0;
                        for (size_t t = 0; t < QK; ++t) idot += (int32_t)aq[r * k + kb * QK + t] * wq[t];
                        cacc += ((float)idot * block_scale(bp)) * as[r * nb + kb];  // matmul_q_i8.zig:466
                    }
                    float &dst = c[r * ldc + j];
                    dst = store_c(alpha, pc == 0 ? beta : 1.0f, cacc, dst);
                }
            }
        }
    });
    return 0;
}

int orc_matmul_q_f32a(int dtype, int nt, size_t m, size_t n, size_t k, float alpha, float beta, const float *a, size_t lda,
                      const uint8_t *b, float *c, size_t ldc, int threads) {
    if (dtype != ORC_Q8_0 && dtype != ORC_Q4_0) return -1;
    if (k % QK != 0) return -1;
    if (lda == 0) lda = k;
    if (ldc == 0) ldc = n;
    const size_t bb = dtype == ORC_Q8_0 ? Q8_BYTES : Q4_BYTES;
    const size_t nb = k / QK;
    parallel_for(n, threads, [&](size_t lo, size_t hi) {
        std::vector<float> w(k);
        for (size_t j = lo; j < hi; ++j) {
            for (size_t kb = 0; kb < nb; ++kb) {
                const uint8_t *bp = nt ? b + (j * nb + kb) * bb : b + (kb * n + j) * bb;
                int8_t wq[QK];
                block_codes(dtype, bp, wq);
                const float s = block_scale(bp);
                for (size_t t = 0; t < QK; ++t) w[kb * QK + t] = (float)wq[t] * s;
            }
            for (size_t r = 0; r < m; ++r) {
                double acc = 0.0;
                for (size_t t = 0; t < k; ++t) acc += (double)a[r * lda + t] * (double)w[t];
                float &dst = c[r * ldc + j];
                dst = beta == 0.0f ? (float)((double)alpha * acc) : (float)((double)alpha * acc + (double)beta * dst);
            }
        }
    });
    return 0;
}

// ---------------------------------------------------------------- attention
int orc_attention_f64(const orc_attn_shape *s, const float *q, const void *k, const void *v,
                      const int32_t *positions, const int32_t *kv_lengths, float *out) {
    if (s->h_kv == 0 || s->h_q % s->h_kv != 0) return -1;
    const size_t groups = s->h_q / s->h_kv;
    std::vector<double> sc(s->t_kv);
    for (size_t b = 0; b < s->batch; ++b) {
        const size_t end = kv_lengths ? (size_t)kv_lengths[b] : s->t_kv;
        if (end > s->t_kv) return -1;
        for (size_t l = 0; l < s->l_q; ++l) {
            const size_t pos = positions ? (size_t)positions[b * s->l_q + l] : l;
            size_t lo, hi;
            window_keys(s->win_left, s->win_right, s->win_chunk, pos, end, lo, hi);
            for (size_t h = 0; h < s->h_q; ++h) {
                const size_t hk = h / groups;
                float *o = out + ((b * s->l_q + l) * s->h_q + h) * s->d_v;
                if (hi <= lo) { std::fill(o, o + s->d_v, 0.0f); continue; }
                const float *qr = q + ((b * s->l_q + l) * s->h_q + h) * s->d_k;
                double mx = -std::numeric_limits<double>::infinity();
                for (size_t t = lo; t < hi; ++t) {
                    const size_t kb = ((b * s->t_kv + t) * s->h_kv + hk) * s->d_k;
                    double d = 0.0;
                    for (size_t j = 0; j < s->d_k; ++j) d += (double)qr[j] * (double)kv_at(k, s->kv_dtype, kb + j);
                    d *= (double)s->scale;
                    if (s->soft_cap > 0.0f) d = (double)s->soft_cap * std::tanh(d / (double)s->soft_cap);
                    sc[t] = d;
                    mx = std::max(mx, d);
                }
                double denom = 0.0;
                for (size_t t = lo; t < hi; ++t) { sc[t] = std::exp(sc[t] - mx); denom += sc[t]; }
                std::vector<double> acc(s->d_v, 0.0);
                for (size_t t = lo; t < hi; ++t) {
                    const size_t vb = ((b * s->t_kv + t) * s->h_kv + hk) * s->d_v;
                    for (size_t j = 0; j < s->d_v; ++j) acc[j] += sc[t] * (double)kv_at(v, s->kv_dtype, vb + j);
                }
                for (size_t j = 0; j < s->d_v; ++j) o[j] = (float)(acc[j] / denom);
            }
        }
    }
    return 0;
}

int orc_attention_blocked(const orc_attn_shape *s, const float *q, const void *k, const void *v,
                          const int32_t *positions, const int32_t *kv_lengths, float *out, int segs_in) {
    if (s->h_kv == 0 || s->h_q % s->h_kv != 0) return -1;
    const size_t ROW_BLOCK = 32, KEY_BLOCK = 256;  // registry/attention_registry.zig:19-50
    const size_t groups = s->h_q / s->h_kv;
    const size_t hb = std::min(groups, ROW_BLOCK);              // exec/attention.zig:1361-1364
    const size_t lb = std::max<size_t>(1, ROW_BLOCK / hb);
    const size_t segs = segs_in < 1 ? 1 : (size_t)segs_in;
    const size_t dk = s->d_k, dv = s->d_v;
    for (size_t b = 0; b < s->batch; ++b) {
        const size_t valid_end = kv_lengths ? (size_t)kv_lengths[b] : s->t_kv;
        if (valid_end > s->t_kv) return -1;
        for (size_t hk = 0; hk < s->h_kv; ++hk)
        for (size_t l0 = 0; l0 < s->l_q; l0 += lb)
        for (size_t g0 = 0; g0 < groups; g0 += hb) {
            const size_t l_n = std::min(lb, s->l_q - l0), hq_n = std::min(hb, groups - g0);
            const size_t rows = l_n * hq_n;
            std::vector<size_t> row_l(rows), row_h(rows), lower(rows), upper(rows);
            size_t uni_lo = std::numeric_limits<size_t>::max(), uni_hi = 0, r = 0;
            for (size_t li = 0; li < l_n; ++li) {
                const size_t l = l0 + li;
                const size_t pos = positions ? (size_t)positions[b * s->l_q + l] : l;
                size_t lo, hi;
                window_keys(s->win_left, s->win_right, s->win_chunk, pos, valid_end, lo, hi);
                if (hi > lo) { uni_lo = std::min(uni_lo, lo); uni_hi = std::max(uni_hi, hi); }
                for (size_t hi_ = 0; hi_ < hq_n; ++hi_, ++r) {
                    row_l[r] = l; row_h[r] = hk * groups + g0 + hi_; lower[r] = lo; upper[r] = hi;
                }
            }
            // per segment partial state (segs == 1: the whole range)
            std::vector<float> acc(segs * rows * dv, 0.0f), m_st(segs * rows, -std::numeric_limits<float>::infinity()), l_st(segs * rows, 0.0f);
            if (uni_hi > uni_lo) {
                std::vector<float> qp(rows * dk);
                for (size_t i = 0; i < rows; ++i) {
                    const float *qr = q + ((b * s->l_q + row_l[i]) * s->h_q + row_h[i]) * dk;
                    for (size_t j = 0; j < dk; ++j) qp[i * dk + j] = qr[j] * s->scale;  // exec/attention.zig:711-718
                }
                const size_t span = uni_hi - uni_lo;
                const size_t seg_len = (span + segs - 1) / segs;
                std::vector<float> scores(rows * KEY_BLOCK), m_new(rows);
                for (size_t sg = 0; sg < segs; ++sg) {
                    float *A = acc.data() + sg * rows * dv, *M = m_st.data() + sg * rows, *L = l_st.data() + sg * rows;
                    const size_t t_start = uni_lo + sg * seg_len, t_end = std::min(t_start + seg_len, uni_hi);
                    for (size_t t = t_start; t < t_end;) {
                        const size_t n = std::min(KEY_BLOCK, t_end - t);
                        std::vector<size_t> lo_b(rows), hi_b(rows);
                        bool any = false;
                        for (size_t i = 0; i < rows; ++i) {
                            const size_t lo = lower[i] > t ? std::min(lower[i] - t, n) : 0;
                            const size_t hi = upper[i] > t ? std::min(upper[i] - t, n) : 0;
                            lo_b[i] = lo; hi_b[i] = hi > lo ? hi : lo;
                            if (hi > lo) any = true;
                        }
                        if (any) {
                            for (size_t i = 0; i < rows; ++i)
                                for (size_t c = 0; c < n; ++c) {
                                    const size_t kb = ((b * s->t_kv + t + c) * s->h_kv + hk) * dk;
                                    float d = 0.0f;
                                    for (size_t j = 0; j < dk; ++j) d += qp[i * dk + j] * kv_at(k, s->kv_dtype, kb + j);
                                    scores[i * n + c] = d;
                                }
                            if (s->soft_cap > 0.0f) {
                                const float inv_cap = 1.0f / s->soft_cap;
                                for (size_t i = 0; i < rows; ++i)
                                    for (size_t c = lo_b[i]; c < hi_b[i]; ++c) scores[i * n + c] = s->soft_cap * tanh_approx(scores[i * n + c] * inv_cap);
                            }
                            for (size_t i = 0; i < rows; ++i) {
                                float mx = M[i];
                                for (size_t c = lo_b[i]; c < hi_b[i]; ++c) mx = std::max(mx, scores[i * n + c]);
                                m_new[i] = mx;
                                const float resc = M[i] == -std::numeric_limits<float>::infinity() ? 1.0f : exp_softmax(M[i] - m_new[i]);
                                L[i] *= resc;
                                if (resc != 1.0f) for (size_t j = 0; j < dv; ++j) A[i * dv + j] *= resc;
                                float ssum = 0.0f;
                                for (size_t c = 0; c < n; ++c) {
                                    if (c < lo_b[i] || c >= hi_b[i]) { scores[i * n + c] = 0.0f; continue; }
                                    const float p = exp_approx(clampf(scores[i * n + c] - mx, -80.0f, 0.0f));
                                    scores[i * n + c] = p;
                                    ssum += p;
                                }
                                L[i] += ssum;
                                for (size_t c = 0; c < n; ++c) {
                                    const float p = scores[i * n + c];
                                    if (p == 0.0f) continue;
                                    const size_t vb = ((b * s->t_kv + t + c) * s->h_kv + hk) * dv;
                                    for (size_t j = 0; j < dv; ++j) A[i * dv + j] += p * kv_at(v, s->kv_dtype, vb + j);
                                }
                                M[i] = m_new[i];
                            }
                        }
                        t += n;
                    }
                }
            }
            // exec/attention.zig:879-962 merge (log-sum-exp over segments), then finalize :787-815
            for (size_t i = 0; i < rows; ++i) {
                float *o = out + ((b * s->l_q + row_l[i]) * s->h_q + row_h[i]) * dv;
                if (upper[i] <= lower[i]) { std::fill(o, o + dv, 0.0f); continue; }
                float m_all = -std::numeric_limits<float>::infinity();
                for (size_t sg = 0; sg < segs; ++sg) m_all = std::max(m_all, m_st[sg * rows + i]);
                float l_all = 0.0f;
                std::vector<float> a_all(dv, 0.0f);
                for (size_t sg = 0; sg < segs; ++sg) {
                    const float ms = m_st[sg * rows + i];
                    if (ms == -std::numeric_limits<float>::infinity()) continue;
                    const float w = segs == 1 ? 1.0f : exp_softmax(ms - m_all);
                    l_all += l_st[sg * rows + i] * w;
                    for (size_t j = 0; j < dv; ++j) a_all[j] += acc[(sg * rows + i) * dv + j] * w;
                }
                if (!(l_all > 0.0f) || !std::isfinite(l_all)) return -1;
                const float inv = 1.0f / l_all;
                for (size_t j = 0; j < dv; ++j) o[j] = a_all[j] * inv;
            }
        }
    }
    return 0;
}

// ---------------------------------------------------------------- glue
void orc_rmsnorm(const float *x, const float *gamma, const float *beta, const float *residual,
                 size_t rows, size_t cols, float eps, float *out) {
    const float inv_denom = 1.0f / (float)cols;
    for (size_t r = 0; r < rows; ++r) {
        const float *xr = x + r * cols;
        float sumsq = 0.0f;
        for (size_t c = 0; c < cols; ++c) sumsq += xr[c] * xr[c];
        const float inv = 1.0f / std::sqrt(sumsq * inv_denom + eps);
        for (size_t c = 0; c < cols; ++c) {
            float y = (xr[c] * inv) * gamma[c] + (beta ? beta[c] : 0.0f);
            if (residual) y += residual[r * cols + c];
            out[r * cols + c] = y;
        }
    }
}

void orc_rope(const float *x, const int32_t *positions, size_t nb, size_t nt, size_t nh, size_t d,
              float base, float scale_factor, float proportion, float *out) {
    const size_t pairs_total = d / 2;
    size_t rope_pairs = (size_t)std::floor(proportion * (float)pairs_total);
    rope_pairs = std::min(rope_pairs, pairs_total);
    const float freq_step = (float)std::pow((double)base, (double)(-2.0f / (float)d));  // exec/rope.zig:50
    for (size_t b = 0; b < nb; ++b)
        for (size_t t = 0; t < nt; ++t) {
            const float pos = (float)positions[b * nt + t];
            const size_t row0 = (b * nt + t) * nh * d;
            std::memcpy(out + row0, x + row0, nh * d * sizeof(float));
            float f = scale_factor;
            for (size_t i = 0; i < rope_pairs; ++i) {
                const float ang = pos * f;
                const float cs = (float)std::cos((double)ang), sn = (float)std::sin((double)ang);
                f *= freq_step;
                for (size_t h = 0; h < nh; ++h) {
                    const float xl = x[row0 + h * d + i], xr = x[row0 + h * d + pairs_total + i];
                    out[row0 + h * d + i] = xl * cs - xr * sn;
                    out[row0 + h * d + pairs_total + i] = xl * sn + xr * cs;
                }
            }
        }
}

void orc_gate_gelu(const float *a, const float *b, size_t n, float *out) {
    for (size_t i = 0; i < n; ++i) {
        const float x = a[i];
        const float t = 0.7978845608028654f * (x + 0.044715f * (x * x * x));
        out[i] = (0.5f * x * (1.0f + tanh_approx(t))) * b[i];
    }
}

// cpu/exec/unary.zig:55-64 over cpu/kernels/{relu,gelu,silu,sigmoid,tanh}.zig; op ids of backend/types.zig:119-125
int orc_unary(int op, const float *x, size_t n, float *out) {
    for (size_t i = 0; i < n; ++i) {
        const float v = x[i];
        switch (op) {
        case 0: out[i] = v > 0.0f ? v : 0.0f; break;
        case 1: out[i] = 0.5f * v * (1.0f + tanh_approx(0.7978845608028654f * (v + 0.044715f * (v * v * v)))); break;
        case 2: out[i] = v * sigmoid_approx(v); break;
        case 3: out[i] = sigmoid_approx(v); break;
        case 4: out[i] = tanh_approx(v); break;
        case 5: out[i] = std::sqrt(v); break;
        default: return -1;
        }
    }
    return 0;
}

// cpu/exec/elementwise.zig:38-60: same shape, scalar b, or b a contiguous suffix of a's shape; op ids of backend/types.zig:92-96
int orc_binary(int op, const float *a, const float *b, size_t n, size_t nb, float *out) {
    if (nb == 0 || n % nb != 0 || op < 0 || op > 3) return -1;
    for (size_t i = 0; i < n; ++i) {
        const float x = a[i], y = b[i % nb];
        out[i] = op == 0 ? x + y : op == 1 ? x - y : op == 2 ? x * y : x / y;
    }
    return 0;
}

void orc_gather_rows(int dtype, const void *table, size_t d, const int32_t *ids, size_t n_ids, float *out) {
    for (size_t i = 0; i < n_ids; ++i) {
        const size_t row = (size_t)ids[i];
        if (dtype == 0) { std::memcpy(out + i * d, (const float *)table + row * d, d * sizeof(float)); continue; }
        const uint8_t *blk = (const uint8_t *)table + row * (d / QK) * Q8_BYTES;
        for (size_t kb = 0; kb < d / QK; ++kb) {
            const float s = block_scale(blk + kb * Q8_BYTES);
            for (size_t t = 0; t < QK; ++t) out[i * d + kb * QK + t] = (float)(int8_t)blk[kb * Q8_BYTES + 2 + t] * s;
        }
    }
}

void orc_argmax(const float *x, size_t rows, size_t n, int32_t *out) {
    for (size_t r = 0; r < rows; ++r) {
        size_t best = 0;
        float bv = x[r * n];
        for (size_t j = 1; j < n; ++j) if (x[r * n + j] > bv) { bv = x[r * n + j]; best = j; }
        out[r] = (int32_t)best;
    }
}

void orc_cast_f32_f16(const float *x, size_t n, uint16_t *out) {
    for (size_t i = 0; i < n; ++i) out[i] = f32_to_f16_bits(x[i]);
}

// ---------------------------------------------------------------- synthetic decoder
// Steps per token block [1,S] (pattern of src/bench/models.zig:433-536 trimmed to a plain
// pre-norm decoder): gather embed -> per layer: rmsnorm -> q,k,v matmul -> rope(q,k) ->
// cast k,v to f16 + append at pos -> causal GQA attention over the cache -> o matmul ->
// add -> rmsnorm -> gate,up matmul -> gelu(gate)*up -> down matmul -> add; then rmsnorm ->
// lm_head matmul -> argmax.
struct orc_decoder {
    orc_decoder_cfg cfg;
    int threads;
    std::map<std::string, std::vector<uint8_t>> w;
    std::vector<std::vector<uint16_t>> kc, vc;  // per layer [max_seq, kv_heads, head_dim] f16
    const std::vector<uint8_t> *get(const std::string &n) const {
        auto it = w.find(n);
        return it == w.end() ? nullptr : &it->second;
    }
    int matmul(const std::string &name, size_t m, size_t n, size_t k, const float *a, float *c) const {
        const auto *b = get(name);
        if (!b) return -1;
        if (cfg.wdtype == ORC_Q8_0) return orc_matmul_nt_q8(m, n, k, 1.0f, 0.0f, a, k, b->data(), c, n, threads);
        return orc_matmul_q_packed(ORC_Q4_0, m, n, k, 1.0f, 0.0f, a, k, b->data(), c, n, 256, threads);
    }
};

orc_decoder *orc_decoder_create(const orc_decoder_cfg *cfg, int threads) {
    auto *d = new orc_decoder();
    d->cfg = *cfg;
    d->threads = threads;
    d->kc.assign(cfg->layers, std::vector<uint16_t>(cfg->max_seq * cfg->kv_heads * cfg->head_dim, 0));
    d->vc = d->kc;
    return d;
}
void orc_decoder_destroy(orc_decoder *d) { delete d; }
int orc_decoder_set_weight(orc_decoder *d, const char *name, const void *data, size_t bytes) {
    d->w[name].assign((const uint8_t *)data, (const uint8_t *)data + bytes);
    return 0;
}
void orc_decoder_reset(orc_decoder *d) {
    for (auto &c : d->kc) std::fill(c.begin(), c.end(), 0);
    for (auto &c : d->vc) std::fill(c.begin(), c.end(), 0);
}

int32_t orc_decoder_forward(orc_decoder *d, const int32_t *tokens, size_t s, size_t pos0, float *logits_last) {
    const orc_decoder_cfg &c = d->cfg;
    const size_t H = c.hidden, QD = c.heads * c.head_dim, KD = c.kv_heads * c.head_dim;
    if (pos0 + s > c.max_seq) return -1;
    const auto *embed = d->get("embed");
    if (!embed) return -1;
    std::vector<float> x(s * H), h(s * H), qv(s * QD), kv(s * KD), vv(s * KD), qr(s * QD), kr(s * KD), att(s * QD), o(s * H);
    std::vector<float> gate(s * c.ffn), up(s * c.ffn), act(s * c.ffn);
    std::vector<int32_t> pos(s);
    for (size_t i = 0; i < s; ++i) pos[i] = (int32_t)(pos0 + i);
    orc_gather_rows(0, embed->data(), H, tokens, s, x.data());
    char nm[64];
    auto wname = [&](size_t l, const char *suffix) { std::snprintf(nm, sizeof nm, "l%zu.%s", l, suffix); return std::string(nm); };
    for (size_t l = 0; l < c.layers; ++l) {
        const auto *g1 = d->get(wname(l, "norm1")), *g2 = d->get(wname(l, "norm2"));
        if (!g1 || !g2) return -1;
        orc_rmsnorm(x.data(), (const float *)g1->data(), nullptr, nullptr, s, H, c.eps, h.data());
        if (d->matmul(wname(l, "wq"), s, QD, H, h.data(), qv.data())) return -1;
        if (d->matmul(wname(l, "wk"), s, KD, H, h.data(), kv.data())) return -1;
        if (d->matmul(wname(l, "wv"), s, KD, H, h.data(), vv.data())) return -1;
        orc_rope(qv.data(), pos.data(), 1, s, c.heads, c.head_dim, c.rope_base, 1.0f, 1.0f, qr.data());
        orc_rope(kv.data(), pos.data(), 1, s, c.kv_heads, c.head_dim, c.rope_base, 1.0f, 1.0f, kr.data());
        orc_cast_f32_f16(kr.data(), s * KD, d->kc[l].data() + pos0 * KD);
        orc_cast_f32_f16(vv.data(), s * KD, d->vc[l].data() + pos0 * KD);
        orc_attn_shape as{};
        as.batch = 1; as.l_q = s; as.t_kv = c.max_seq; as.h_q = c.heads; as.h_kv = c.kv_heads; as.d_k = as.d_v = c.head_dim;
        as.scale = 1.0f / std::sqrt((float)c.head_dim); as.soft_cap = 0.0f;
        as.win_left = 0xFFFFFFFFu; as.win_right = 0; as.win_chunk = 0; as.kv_dtype = 1;
        const int32_t end = (int32_t)(pos0 + s);
        if (c.attn_exact) {
            if (orc_attention_f64(&as, qr.data(), d->kc[l].data(), d->vc[l].data(), pos.data(), &end, att.data())) return -1;
        } else if (orc_attention_blocked(&as, qr.data(), d->kc[l].data(), d->vc[l].data(), pos.data(), &end, att.data(), 1)) {
            return -1;
        }
        if (d->matmul(wname(l, "wo"), s, H, QD, att.data(), o.data())) return -1;
        for (size_t i = 0; i < s * H; ++i) x[i] += o[i];
        orc_rmsnorm(x.data(), (const float *)g2->data(), nullptr, nullptr, s, H, c.eps, h.data());
        if (d->matmul(wname(l, "wgate"), s, c.ffn, H, h.data(), gate.data())) return -1;
        if (d->matmul(wname(l, "wup"), s, c.ffn, H, h.data(), up.data())) return -1;
        orc_gate_gelu(gate.data(), up.data(), s * c.ffn, act.data());
        if (d->matmul(wname(l, "wdown"), s, H, c.ffn, act.data(), o.data())) return -1;
        for (size_t i = 0; i < s * H; ++i) x[i] += o[i];
    }
    const auto *gf = d->get("norm_f");
    if (!gf) return -1;
    // only the last row feeds the logits head
    std::vector<float> hl(H), logits(c.vocab);
    orc_rmsnorm(x.data() + (s - 1) * H, (const float *)gf->data(), nullptr, nullptr, 1, H, c.eps, hl.data());
    if (d->matmul("lm_head", 1, c.vocab, H, hl.data(), logits.data())) return -1;
    int32_t best;
    orc_argmax(logits.data(), 1, c.vocab, &best);
    if (logits_last) std::memcpy(logits_last, logits.data(), c.vocab * sizeof(float));
    return best;
}

}  // extern "C"
