// Prefill GEMM back ends (more than 8 activation rows): C[m,n] = alpha * A[m,:] . W[n,:] + beta * C.
//
// gemm_i8_kernel (AIONHIP_GEMM_EXACT_I8) - aion's CPU arithmetic (cpu/kernels/matmul_q_i8.zig:
//   384-497): activations int8 per (row, 32-block), one v_mfma_i32_16x16x32_i8 per 16x16 output
//   tile per quant block (K=32 IS one block, so the i32 tile is the exact block dot), then
//   acc += f32(idot) * (a_scale * w_scale) on the VALU. Operands come straight from global
//   memory in MFMA layout (8 bytes per lane per tile). The per-block rescale (3 VALU ops per
//   output element per block) is what bounds it, not the MFMA pipe.
//
// gemm_bf16_kernel (AIONHIP_GEMM_BF16_MFMA) - weights dequantized once to bf16 [N,K] (kept per
//   weight: 288 GB of HBM makes the 2 B/weight copy affordable), activations rounded to bf16,
//   v_mfma_f32_16x16x32_bf16 with f32 accumulation. Workgroup tile 256x128, K step 32, operands
//   staged through double-buffered LDS (row stride 80 B: conflict-free 16-byte operand reads),
//   global loads of the next K step in flight during the MFMAs of the current one.
#include "common.h"

namespace {

using i32x4 = __attribute__((ext_vector_type(4))) int;
using bf16x8 = __attribute__((ext_vector_type(8))) __bf16;

// ------------------------------------------------------------------------------------ exact int8
template <int DT, int TM>
__global__ __launch_bounds__(256) void gemm_i8_kernel(const uint8_t *__restrict__ qs, const __half *__restrict__ sc,
                                                      const int8_t *__restrict__ aq, const float *__restrict__ a_scale,
                                                      const int *__restrict__ a_sum, float *__restrict__ c,
                                                      int M, int N, int K, size_t ldc, float alpha, float beta) {
    constexpr int TN = 4;
    constexpr bool Q8 = DT == AIONHIP_Q8_0;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int n0 = (blockIdx.x * 4 + wave) * (TN * 16);
    const int m0 = blockIdx.y * (TM * 16);
    if (n0 >= N) return;
    const int KB = K >> 5;

    f32x4 acc[TM][TN];
#pragma unroll
    for (int mi = 0; mi < TM; ++mi)
#pragma unroll
        for (int ni = 0; ni < TN; ++ni) acc[mi][ni] = f32x4{0.f, 0.f, 0.f, 0.f};

    size_t arow[TM], srow[TM][4], wrow[TN];
#pragma unroll
    for (int mi = 0; mi < TM; ++mi) {
        arow[mi] = (size_t)min(m0 + mi * 16 + r, M - 1) * K;
#pragma unroll
        for (int i = 0; i < 4; ++i) srow[mi][i] = (size_t)min(m0 + mi * 16 + g * 4 + i, M - 1) * KB;
    }
#pragma unroll
    for (int ni = 0; ni < TN; ++ni) wrow[ni] = (size_t)min(n0 + ni * 16 + r, N - 1);

    for (int kb = 0; kb < KB; ++kb) {
        long a[TM], b[TN];
        float ws[TN];
#pragma unroll
        for (int mi = 0; mi < TM; ++mi) a[mi] = *(const long *)(aq + arow[mi] + kb * 32 + g * 8);
#pragma unroll
        for (int ni = 0; ni < TN; ++ni) {
            if (Q8) {
                b[ni] = *(const long *)(qs + wrow[ni] * K + kb * 32 + g * 8);
            } else {
                const unsigned w = *(const unsigned *)(qs + wrow[ni] * (K >> 1) + kb * 16 + g * 4);
                b[ni] = (long)(((unsigned long)((w >> 4) & 0x0F0F0F0Fu) << 32) | (unsigned long)(w & 0x0F0F0F0Fu));
            }
            ws[ni] = __half2float(sc[wrow[ni] * KB + kb]);
        }
#pragma unroll
        for (int mi = 0; mi < TM; ++mi) {
            float as[4];
            int bias[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                as[i] = a_scale[srow[mi][i] + kb];
                bias[i] = Q8 ? 0 : 8 * a_sum[srow[mi][i] + kb];
            }
#pragma unroll
            for (int ni = 0; ni < TN; ++ni) {
                const i32x4 d = __builtin_amdgcn_mfma_i32_16x16x32_i8(a[mi], b[ni], i32x4{0, 0, 0, 0}, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[mi][ni][i] += (float)(d[i] - bias[i]) * (as[i] * ws[ni]);
            }
        }
    }

#pragma unroll
    for (int mi = 0; mi < TM; ++mi)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = m0 + mi * 16 + g * 4 + i;
            if (row >= M) continue;
#pragma unroll
            for (int ni = 0; ni < TN; ++ni) {
                const int col = n0 + ni * 16 + r;
                if (col >= N) continue;
                float *dst = c + (size_t)row * ldc + col;
                const float v = alpha * acc[mi][ni][i];
                *dst = beta == 0.f ? v : v + beta * *dst;
            }
        }
}

// ------------------------------------------------------------------------------------ bf16 MFMA
__device__ __forceinline__ unsigned short bf16_rne(float x) {
    unsigned u = __float_as_uint(x);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
}

// device row layout -> bf16 [N][K]: value = code * f32(f16 scale), rounded to bf16
template <int DT>
__global__ void dequant_bf16_kernel(const uint8_t *__restrict__ qs, const __half *__restrict__ sc, unsigned short *__restrict__ out,
                                    size_t N, size_t K) {
    // one thread per 8 consecutive k of one row
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t per_row = K / 8;
    if (i >= N * per_row) return;
    const size_t n = i / per_row, k0 = (i % per_row) * 8;
    const float s = __half2float(sc[n * (K / QK) + k0 / QK]);
    int code[8];
    if (DT == AIONHIP_Q8_0) {
        const long v = *(const long *)(qs + n * K + k0);
#pragma unroll
        for (int j = 0; j < 8; ++j) code[j] = (int)(int8_t)(v >> (8 * j));
    } else {
        const unsigned w = *(const unsigned *)(qs + n * (K / 2) + k0 / 2);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            code[j] = (int)((w >> (8 * j)) & 15u) - 8;
            code[4 + j] = (int)((w >> (8 * j + 4)) & 15u) - 8;
        }
    }
    u32x4 o;
    o.x = (unsigned)bf16_rne((float)code[0] * s) | ((unsigned)bf16_rne((float)code[1] * s) << 16);
    o.y = (unsigned)bf16_rne((float)code[2] * s) | ((unsigned)bf16_rne((float)code[3] * s) << 16);
    o.z = (unsigned)bf16_rne((float)code[4] * s) | ((unsigned)bf16_rne((float)code[5] * s) << 16);
    o.w = (unsigned)bf16_rne((float)code[6] * s) | ((unsigned)bf16_rne((float)code[7] * s) << 16);
    *(u32x4 *)(out + n * K + k0) = o;
}

__global__ void act_bf16_kernel(const float *__restrict__ a, size_t lda, unsigned short *__restrict__ out, size_t M, size_t K) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t per_row = K / 8;
    if (i >= M * per_row) return;
    const size_t m = i / per_row, k0 = (i % per_row) * 8;
    const float *p = a + m * lda + k0;
    u32x4 o;
    o.x = (unsigned)bf16_rne(p[0]) | ((unsigned)bf16_rne(p[1]) << 16);
    o.y = (unsigned)bf16_rne(p[2]) | ((unsigned)bf16_rne(p[3]) << 16);
    o.z = (unsigned)bf16_rne(p[4]) | ((unsigned)bf16_rne(p[5]) << 16);
    o.w = (unsigned)bf16_rne(p[6]) | ((unsigned)bf16_rne(p[7]) << 16);
    *(u32x4 *)(out + m * K + k0) = o;
}

// ---- wide-tile kernel: workgroup tile (WM*64) x 256, K step 64, v_mfma_f32_32x32x16_bf16.
// 2 x 2 wavefronts, each (WM*32) x 128 outputs = WM x 4 tiles of 32x32 (accumulators: WM*64
// registers). Operands go global -> registers -> LDS (row stride 144 B: 16 consecutive rows land
// in 16 distinct 16-byte bank groups) -> 16-byte fragment reads; the next K step's global loads
// are in flight during the MFMAs of the current one, one barrier per K step.
// Tile order: workgroup ids go round-robin over the 8 XCDs, so id -> (xcd, slot) -> a contiguous
// run of tiles per XCD, M fastest: the workgroups that share a weight column tile run on one L2.
constexpr int G2_BK = 64, G2_STRIDE = 144, G2_BN = 256;
using f32x16 = __attribute__((ext_vector_type(16))) float;

template <int WM>
__global__ __launch_bounds__(256) void gemm_bf16_wide_kernel(const unsigned short *__restrict__ A, const unsigned short *__restrict__ W,
                                                             float *__restrict__ c, int M, int N, int K, size_t ldc, float alpha,
                                                             float beta, int tiles_m, int tiles) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds2[];
    constexpr int BM2 = WM * 64;
    constexpr int A_BYTES = BM2 * G2_STRIDE, B_BYTES = G2_BN * G2_STRIDE, STAGE = A_BYTES + B_BYTES;
    constexpr int NA = WM * 2, NB = 8;                       // 16-byte chunks per thread per stage
    const int per_xcd = (int)gridDim.x >> 3;
    const int t = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
    if (t >= tiles) return;
    const int m0 = (t % tiles_m) * BM2, n0 = (t / tiles_m) * G2_BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l31 = lane & 31, lh = lane >> 5;
    const int wrow = (wave >> 1) * (WM * 32), wcol = (wave & 1) * 128;

    f32x16 acc[WM][4];
#pragma unroll
    for (int mi = 0; mi < WM; ++mi)
#pragma unroll
        for (int ni = 0; ni < 4; ++ni)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mi][ni][i] = 0.f;

    const unsigned short *ga[NA], *gb[NB];
    int la[NA], lb[NB];
#pragma unroll
    for (int i = 0; i < NA; ++i) {
        const int ch = tid + 256 * i, row = ch >> 3, part = ch & 7;
        ga[i] = A + (size_t)min(m0 + row, M - 1) * K + part * 8;
        la[i] = row * G2_STRIDE + part * 16;
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        const int ch = tid + 256 * i, row = ch >> 3, part = ch & 7;
        gb[i] = W + (size_t)min(n0 + row, N - 1) * K + part * 8;
        lb[i] = A_BYTES + row * G2_STRIDE + part * 16;
    }
    const int fa = (wrow + l31) * G2_STRIDE + lh * 16;              // + mi * 32 rows + ks * 32 bytes
    const int fb = A_BYTES + (wcol + l31) * G2_STRIDE + lh * 16;

    const int KT = K / G2_BK;
    u32x4 ra[NA], rb[NB];
#pragma unroll
    for (int i = 0; i < NA; ++i) ra[i] = *(const u32x4 *)(ga[i]);
#pragma unroll
    for (int i = 0; i < NB; ++i) rb[i] = *(const u32x4 *)(gb[i]);
#pragma unroll
    for (int i = 0; i < NA; ++i) *(u32x4 *)(lds2 + la[i]) = ra[i];
#pragma unroll
    for (int i = 0; i < NB; ++i) *(u32x4 *)(lds2 + lb[i]) = rb[i];
    __syncthreads();

    // Software pipeline, one basic block per K step so that the instruction groups can be pinned:
    //   sub-step 0: global loads of the next K step + MFMAs(0) while the fragments of sub-step 1 are read
    //   sub-step 1: MFMAs(1) while fragments 2 are read;  sub-step 2: MFMAs(2) while fragments 3 are read
    //   staged registers -> the other LDS buffer, barrier
    //   sub-step 3: MFMAs(3) while fragments 0 of the next K step are read from the other buffer
    // The last K step repeats its own loads into the idle buffer instead of branching.
    struct Frag {
        u32x4 a[WM], b[4];
    };
    auto read_frag = [&](Frag &f, const unsigned char *st, int ks) {
#pragma unroll
        for (int ni = 0; ni < 4; ++ni) f.b[ni] = *(const u32x4 *)(st + fb + ni * 32 * G2_STRIDE + ks * 32);
#pragma unroll
        for (int mi = 0; mi < WM; ++mi) f.a[mi] = *(const u32x4 *)(st + fa + mi * 32 * G2_STRIDE + ks * 32);
    };
    auto mma = [&](const Frag &f) {
#pragma unroll
        for (int mi = 0; mi < WM; ++mi)
#pragma unroll
            for (int ni = 0; ni < 4; ++ni)
                acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, f.a[mi]), __builtin_bit_cast(bf16x8, f.b[ni]), acc[mi][ni], 0, 0, 0);
    };
    constexpr int NMMA = WM * 4, NFR = WM + 4;
    Frag f0, f1;
    read_frag(f0, lds2, 0);
    for (int kt = 0; kt < KT; ++kt) {
        const unsigned char *st = lds2 + (kt & 1) * STAGE;
        unsigned char *nx = lds2 + ((kt + 1) & 1) * STAGE;
        const size_t knext = (size_t)min(kt + 1, KT - 1) * G2_BK;
#pragma unroll
        for (int i = 0; i < NA; ++i) ra[i] = *(const u32x4 *)(ga[i] + knext);
#pragma unroll
        for (int i = 0; i < NB; ++i) rb[i] = *(const u32x4 *)(gb[i] + knext);
        read_frag(f1, st, 1);
        mma(f0);
        // one global load then one MFMA, NA + NB times; the fragment reads spread over the MFMAs
#pragma unroll
        for (int i = 0; i < NFR; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x020, (NA + NB) / NFR, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, NMMA / NFR, 0);
        }
        read_frag(f0, st, 2);
        mma(f1);
#pragma unroll
        for (int i = 0; i < NFR; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, NMMA / NFR, 0);
        }
        read_frag(f1, st, 3);
        mma(f0);
#pragma unroll
        for (int i = 0; i < NFR; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, NMMA / NFR, 0);
        }
#pragma unroll
        for (int i = 0; i < NA; ++i) *(u32x4 *)(nx + la[i]) = ra[i];
#pragma unroll
        for (int i = 0; i < NB; ++i) *(u32x4 *)(nx + lb[i]) = rb[i];
        __syncthreads();
        read_frag(f0, nx, 0);
        mma(f1);
#pragma unroll
        for (int i = 0; i < NFR; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, NMMA / NFR, 0);
        }
    }

    // 32x32 accumulator layout: element i of lane l is row (i / 4) * 8 + (l / 32) * 4 + i % 4, column l % 32
#pragma unroll
    for (int mi = 0; mi < WM; ++mi)
#pragma unroll
        for (int ni = 0; ni < 4; ++ni) {
            const int col = n0 + wcol + ni * 32 + l31;
            if (col >= N) continue;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int row = m0 + wrow + mi * 32 + (i >> 2) * 8 + lh * 4 + (i & 3);
                if (row >= M) continue;
                float *dst = c + (size_t)row * ldc + col;
                const float v = alpha * acc[mi][ni][i];
                *dst = beta == 0.f ? v : v + beta * *dst;
            }
        }
}

constexpr int BM = 256, BN = 128, BK = 32;
constexpr int LDS_ROW = 80;                       // 64 B of bf16 + 16 B pad
constexpr int A_TILE = BM * LDS_ROW, B_TILE = BN * LDS_ROW;

__global__ __launch_bounds__(256) void gemm_bf16_kernel(const unsigned short *__restrict__ A, const unsigned short *__restrict__ W,
                                                        float *__restrict__ c, int M, int N, int K, size_t ldc, float alpha, float beta) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * (A_TILE + B_TILE)];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int wm0 = (wave >> 1) * 128, wn0 = (wave & 1) * 64;   // 2 x 2 wavefronts, each 128 x 64
    constexpr int TM = 8, TN = 4;

    f32x4 acc[TM][TN];
#pragma unroll
    for (int mi = 0; mi < TM; ++mi)
#pragma unroll
        for (int ni = 0; ni < TN; ++ni) acc[mi][ni] = f32x4{0.f, 0.f, 0.f, 0.f};

    // global -> LDS assignment: 16-byte chunks; A tile 1024 chunks (4 per thread), B tile 512 (2 per thread)
    const unsigned short *ga[4];
    const unsigned short *gb[2];
    int la[4], lb[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int ch = tid + 256 * i, row = ch >> 2, part = ch & 3;
        ga[i] = A + (size_t)min(m0 + row, M - 1) * K + part * 8;
        la[i] = row * LDS_ROW + part * 16;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int ch = tid + 256 * i, row = ch >> 2, part = ch & 3;
        gb[i] = W + (size_t)min(n0 + row, N - 1) * K + part * 8;
        lb[i] = row * LDS_ROW + part * 16;
    }

    const int KT = K / BK;
    u32x4 ra[4], rb[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) ra[i] = *(const u32x4 *)(ga[i]);
#pragma unroll
    for (int i = 0; i < 2; ++i) rb[i] = *(const u32x4 *)(gb[i]);
#pragma unroll
    for (int i = 0; i < 4; ++i) *(u32x4 *)(lds + la[i]) = ra[i];
#pragma unroll
    for (int i = 0; i < 2; ++i) *(u32x4 *)(lds + A_TILE + lb[i]) = rb[i];
    __syncthreads();

    for (int kt = 0; kt < KT; ++kt) {
        const unsigned char *sa = lds + (kt & 1) * (A_TILE + B_TILE);
        const unsigned char *sb = sa + A_TILE;
        const bool more = kt + 1 < KT;
        if (more) {
#pragma unroll
            for (int i = 0; i < 4; ++i) ra[i] = *(const u32x4 *)(ga[i] + (size_t)(kt + 1) * BK);
#pragma unroll
            for (int i = 0; i < 2; ++i) rb[i] = *(const u32x4 *)(gb[i] + (size_t)(kt + 1) * BK);
        }
        u32x4 bf[TN];
#pragma unroll
        for (int ni = 0; ni < TN; ++ni) bf[ni] = *(const u32x4 *)(sb + (wn0 + ni * 16 + r) * LDS_ROW + g * 16);
#pragma unroll
        for (int mi = 0; mi < TM; ++mi) {
            const u32x4 af = *(const u32x4 *)(sa + (wm0 + mi * 16 + r) * LDS_ROW + g * 16);
#pragma unroll
            for (int ni = 0; ni < TN; ++ni)
                acc[mi][ni] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, af), __builtin_bit_cast(bf16x8, bf[ni]), acc[mi][ni], 0, 0, 0);
        }
        if (more) {
            unsigned char *da = lds + ((kt + 1) & 1) * (A_TILE + B_TILE);
#pragma unroll
            for (int i = 0; i < 4; ++i) *(u32x4 *)(da + la[i]) = ra[i];
#pragma unroll
            for (int i = 0; i < 2; ++i) *(u32x4 *)(da + A_TILE + lb[i]) = rb[i];
        }
        __syncthreads();
    }

#pragma unroll
    for (int mi = 0; mi < TM; ++mi)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = m0 + wm0 + mi * 16 + g * 4 + i;
            if (row >= M) continue;
#pragma unroll
            for (int ni = 0; ni < TN; ++ni) {
                const int col = n0 + wn0 + ni * 16 + r;
                if (col >= N) continue;
                float *dst = c + (size_t)row * ldc + col;
                const float v = alpha * acc[mi][ni][i];
                *dst = beta == 0.f ? v : v + beta * *dst;
            }
        }
}

template <int DT>
void launch_i8(aionhip_ctx *ctx, const aionhip_weight *w, size_t m, PreparedAct act, float *c, size_t ldc, float alpha, float beta) {
    const int M = (int)m, N = (int)w->n, K = (int)w->k;
    const unsigned gx = (unsigned)((N + 255) / 256);
    if (M > 32) {
        launch_k(ctx, gemm_i8_kernel<DT, 4>, dim3(gx, (unsigned)((M + 63) / 64)), dim3(256), 0, w->qs, w->sc, act.q, act.scale, act.sum, c, M, N, K, ldc, alpha, beta);
    } else if (M > 16) {
        launch_k(ctx, gemm_i8_kernel<DT, 2>, dim3(gx, (unsigned)((M + 31) / 32)), dim3(256), 0, w->qs, w->sc, act.q, act.scale, act.sum, c, M, N, K, ldc, alpha, beta);
    } else {
        launch_k(ctx, gemm_i8_kernel<DT, 1>, dim3(gx, (unsigned)((M + 15) / 16)), dim3(256), 0, w->qs, w->sc, act.q, act.scale, act.sum, c, M, N, K, ldc, alpha, beta);
    }
}

}  // namespace

int launch_gemm_i8(aionhip_ctx *ctx, const aionhip_weight *w, size_t m, PreparedAct act, float *c, size_t ldc, float alpha, float beta) {
    const char *name = w->dtype == AIONHIP_Q8_0 ? "gemm_i8_q8" : "gemm_i8_q4";
    ProfScope scope(ctx, name);
    if (w->dtype == AIONHIP_Q8_0) launch_i8<AIONHIP_Q8_0>(ctx, w, m, act, c, ldc, alpha, beta);
    else launch_i8<AIONHIP_Q4_0>(ctx, w, m, act, c, ldc, alpha, beta);
    LAUNCH_CHECK(ctx, name);
    return AIONHIP_OK;
}

int launch_gemm_bf16(aionhip_ctx *ctx, const aionhip_weight *cw, size_t m, const float *a, size_t lda, float *c, size_t ldc, float alpha, float beta) {
    aionhip_weight *w = const_cast<aionhip_weight *>(cw);   // the bf16 copy is a cache on the weight
    const size_t N = w->n, K = w->k;
    if ((((uintptr_t)a) & 3) != 0) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "gemm: A must be 4-byte aligned");
    if (!w->bf16) {
        void *p = nullptr;
        HIP_TRY(ctx, hipMalloc(&p, N * K * 2));
        w->bf16 = (unsigned short *)p;
        const size_t threads = N * (K / 8);
        const unsigned grid = (unsigned)((threads + 255) / 256);
        if (w->dtype == AIONHIP_Q8_0) dequant_bf16_kernel<AIONHIP_Q8_0><<<dim3(grid), dim3(256), 0, ctx->stream>>>(w->qs, w->sc, w->bf16, N, K);
        else dequant_bf16_kernel<AIONHIP_Q4_0><<<dim3(grid), dim3(256), 0, ctx->stream>>>(w->qs, w->sc, w->bf16, N, K);
        LAUNCH_CHECK(ctx, "dequant_bf16");
    }
    int rc = ensure_scratch2(ctx, m * K * 2);
    if (rc) return rc;
    unsigned short *abf = (unsigned short *)ctx->scratch2;
    {
        const size_t threads = m * (K / 8);
        ProfScope scope(ctx, "act_bf16");
        launch_k(ctx, act_bf16_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, a, lda, abf, m, K);
        LAUNCH_CHECK(ctx, "act_bf16");
    }
    ProfScope scope(ctx, "gemm_bf16");
    if (K % G2_BK == 0) {
        // 256-row tiles when they still give every CU a workgroup, else 128-row tiles
        const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
        const int tn = (int)((N + G2_BN - 1) / G2_BN);
        const int tm4 = (int)((m + 255) / 256), tm2 = (int)((m + 127) / 128);
        const bool big = (long)tm4 * tn >= cus;
        const int tm = big ? tm4 : tm2, tiles = tm * tn;
        const dim3 grid((unsigned)((tiles + 7) / 8 * 8));
        static bool attr4 = false, attr2 = false;
        if (big) {
            constexpr int LDS = 2 * (256 + G2_BN) * G2_STRIDE;
            if (!attr4) {
                HIP_TRY(ctx, hipFuncSetAttribute((const void *)gemm_bf16_wide_kernel<4>, hipFuncAttributeMaxDynamicSharedMemorySize, LDS));
                attr4 = true;
            }
            launch_k(ctx, gemm_bf16_wide_kernel<4>, grid, dim3(256), LDS, abf, w->bf16, c, (int)m, (int)N, (int)K, ldc, alpha, beta, tm, tiles);
        } else {
            constexpr int LDS = 2 * (128 + G2_BN) * G2_STRIDE;
            if (!attr2) {
                HIP_TRY(ctx, hipFuncSetAttribute((const void *)gemm_bf16_wide_kernel<2>, hipFuncAttributeMaxDynamicSharedMemorySize, LDS));
                attr2 = true;
            }
            launch_k(ctx, gemm_bf16_wide_kernel<2>, grid, dim3(256), LDS, abf, w->bf16, c, (int)m, (int)N, (int)K, ldc, alpha, beta, tm, tiles);
        }
    } else {
        const dim3 grid((unsigned)((N + BN - 1) / BN), (unsigned)((m + BM - 1) / BM));
        launch_k(ctx, gemm_bf16_kernel, grid, dim3(256), 0, abf, w->bf16, c, (int)m, (int)N, (int)K, ldc, alpha, beta);
    }
    LAUNCH_CHECK(ctx, "gemm_bf16");
    return AIONHIP_OK;
}
