// Prefill GEMM back ends (more than 8 activation rows): C[m,n] = alpha * A[m,:] . W[n,:] + beta * C.
//
// gemm_i8_lds_kernel (AIONHIP_GEMM_EXACT_I8) - aion's CPU arithmetic (cpu/kernels/matmul_q_i8.zig:
//   384-497): activations int8 per (row, 32-block), one v_mfma_i32_16x16x32_i8 per 16x16 output
//   tile per quant block (K=32 IS one block, so the i32 tile is the exact block dot), then
//   acc += f32(idot) * (a_scale * w_scale) on the VALU. Operands are staged through LDS. The per-block
//   rescale (3 VALU ops per output element per block) is what bounds it, not the MFMA pipe.
//
// gemm_bf16_wide_kernel (AIONHIP_GEMM_BF16_MFMA) - weights as bf16, either from a copy the context builds once per
//   weight and owns (2 B/weight; 288 GB of HBM makes it affordable) or converted from the quant blocks while they are
//   staged (no copy; same bits, slower), activations rounded to bf16, v_mfma_f32_32x32x16_bf16 with f32 accumulation;
//   described at the kernel.
#include "common.h"

#include <type_traits>
#include <utility>

namespace {

using u32x2 = __attribute__((ext_vector_type(2))) unsigned int;
using i32x4 = __attribute__((ext_vector_type(4))) int;
using bf16x8 = __attribute__((ext_vector_type(8))) __bf16;

// ------------------------------------------------------------------------------------ exact int8
// ---- LDS-staged exact kernel: one
// v_mfma_i32_16x16x32_i8 per 16x16 tile per quant block, then acc += f32(idot) * (a_scale * w_scale) - but
// the operands of a K step (4 quant blocks) are staged once per workgroup in LDS with coalesced 16-byte
// loads (a cache line per row), instead of 8-byte operand loads per lane per tile from global memory, which
// cost several times their payload in L1 bandwidth. q4 nibbles become signed int8 while they are staged
// (((x | 0x80) - 8) ^ 0x80 per byte), so no per-tile bias correction is left. Workgroup tile (32*WM) x 128,
// 2 x 2 wavefronts of (16*WM) x 64 outputs; double-buffered, one barrier per K step. The rescale (3 VALU
// operations per output per block against 32 integer MACs) bounds it at roughly 1/7 of the int8 MFMA peak.
// KC = quant blocks per K step: 4 when the grid fills the device (two workgroups per CU hide each other's
// staging), 8 when it does not (few activation rows: fewer, larger steps - a step then costs one memory
// latency however little it loads).
// up to four weights with the same K and block format against one prepared activation: column tiles first_tile[i] .. of weight i
struct GemmSegs {
    const uint8_t *qs[4];
    const __half *sc[4];
    float *c[4];
    size_t ldc[4];
    int n[4], first_tile[4];
    int count;
};
template <int KC> struct GiCfg { static constexpr int ROW = KC * 32 + 16; };   // staged code row; +16 B: conflict-free 8-byte operand reads
// SPLITK (few activation rows, where the tiles above would leave most CUs idle): the workgroup tile shrinks
// to (16*WM) x 64 and its four wavefronts share it, each taking every fourth quant block of a K step; their
// partial sums are added in wavefront order through LDS at the end, so the result does not depend on timing.
template <int DT, int WM, int KC, bool SPLITK>
__global__ __launch_bounds__(256, KC == 4 || SPLITK ? 2 : 1) void gemm_i8_lds_kernel(GemmSegs segs,
                                                          const int8_t *__restrict__ aq, const float *__restrict__ a_scale,
                                                          int M, int K, float alpha, float beta, float *__restrict__ partial, int partial_ld) {
    constexpr bool Q8 = DT == AIONHIP_Q8_0;
    static_assert(!SPLITK || KC == 8, "split K: two blocks per wavefront per step");
    constexpr int BM3 = (SPLITK ? 16 : 32) * WM, BN3 = SPLITK ? 64 : 128, ROW = GiCfg<KC>::ROW;
    constexpr int KCW = SPLITK ? KC / 4 : KC;            // blocks of a K step this wavefront works on
    constexpr int A_BYTES = BM3 * ROW, B_BYTES = BN3 * ROW;
    constexpr int AS_BYTES = BM3 * KC * 4, WS_BYTES = BN3 * KC * 4;
    constexpr int STAGE = A_BYTES + B_BYTES + AS_BYTES + WS_BYTES;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds3[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4;
    // the weight this column tile belongs to (sibling weights over one activation share a launch)
    int si = 0;
#pragma unroll
    for (int i = 1; i < 4; ++i)
        if (i < segs.count && (int)blockIdx.x >= segs.first_tile[i]) si = i;
    const uint8_t *__restrict__ qs = segs.qs[si];
    const __half *__restrict__ sc = segs.sc[si];
    float *__restrict__ c = segs.c[si];
    const int N = segs.n[si];
    const size_t ldc = segs.ldc[si];
    const int m0 = blockIdx.y * BM3, n0 = ((int)blockIdx.x - segs.first_tile[si]) * BN3;
    const int wm0 = SPLITK ? 0 : (wave >> 1) * (16 * WM), wn0 = SPLITK ? 0 : (wave & 1) * 64;
    const int jw = SPLITK ? wave : 0, jstep = SPLITK ? 4 : 1;     // this wavefront's blocks: jw + jstep * jj
    const int KB = K >> 5, KT = (KB + KC - 1) / KC;

    f32x4 acc[WM][4];
#pragma unroll
    for (int mi = 0; mi < WM; ++mi)
#pragma unroll
        for (int ni = 0; ni < 4; ++ni) acc[mi][ni] = f32x4{0.f, 0.f, 0.f, 0.f};

    // staging assignment: 16-byte chunks, 2*KC per code row of a K step (q4 weights: KC, one block each)
    constexpr int CPR = 2 * KC;                          // chunks per int8 row
    constexpr int NAC = BM3 * CPR / 256;                 // activation chunks per thread
    constexpr int NBC = (Q8 ? BN3 * CPR : BN3 * KC) / 256;
    constexpr int NAS = (BM3 * KC + 255) / 256, NWS = BN3 * KC / 256;
    u32x4 ra[NAC], rb[NBC];
    float ras[NAS];
    __half rws[NWS];                                     // converted when stored: a conversion here would wait for the load
    auto load_stage = [&](int kt) {
        const int kb0 = kt * KC;
#pragma unroll
        for (int i = 0; i < NAC; ++i) {
            const int id = tid + 256 * i, row = id / CPR, part = id % CPR;
            const int kbyte = min(kb0 * 32 + part * 16, K - 16);
            ra[i] = *(const u32x4 *)(aq + (size_t)min(m0 + row, M - 1) * K + kbyte);
        }
#pragma unroll
        for (int i = 0; i < NBC; ++i) {
            const int id = tid + 256 * i;
            if (Q8) {
                const int row = id / CPR, part = id % CPR;
                const int kbyte = min(kb0 * 32 + part * 16, K - 16);
                rb[i] = *(const u32x4 *)(qs + (size_t)min(n0 + row, N - 1) * K + kbyte);
            } else {
                const int row = id / KC, blk = min(kb0 + id % KC, KB - 1);
                rb[i] = *(const u32x4 *)(qs + (size_t)min(n0 + row, N - 1) * (K >> 1) + (size_t)blk * 16);
            }
        }
#pragma unroll
        for (int i = 0; i < NAS; ++i) {
            // unconditional loads at clamped addresses (a predicated load is waited for on the spot)
            const int id = min(tid + 256 * i, BM3 * KC - 1), row = id / KC, j = id % KC;
            ras[i] = a_scale[(size_t)min(m0 + row, M - 1) * KB + min(kb0 + j, KB - 1)];
        }
#pragma unroll
        for (int i = 0; i < NWS; ++i) {
            const int id = tid + 256 * i, row = id / KC, j = id % KC;
            rws[i] = sc[(size_t)min(n0 + row, N - 1) * KB + min(kb0 + j, KB - 1)];
        }
    };
    auto store_stage = [&](unsigned char *st, int kt) {
        const int kb0 = kt * KC;
#pragma unroll
        for (int i = 0; i < NAC; ++i) {
            const int id = tid + 256 * i, row = id / CPR, part = id % CPR;
            *(u32x4 *)(st + row * ROW + part * 16) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < NBC; ++i) {
            const int id = tid + 256 * i;
            if (Q8) {
                const int row = id / CPR, part = id % CPR;
                *(u32x4 *)(st + A_BYTES + row * ROW + part * 16) = rb[i];
            } else {
                // word w of the device layout holds elements 8w..8w+7: low nibbles 8w..8w+3, high nibbles 8w+4..8w+7
                const int row = id / KC, j = id % KC;
                unsigned char *dst = st + A_BYTES + row * ROW + j * 32;
                const unsigned ws4[4] = {rb[i].x, rb[i].y, rb[i].z, rb[i].w};
                unsigned dec[8];
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const unsigned lo = ws4[w] & 0x0F0F0F0Fu, hi = (ws4[w] >> 4) & 0x0F0F0F0Fu;
                    dec[2 * w] = ((lo | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
                    dec[2 * w + 1] = ((hi | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
                }
                *(u32x4 *)dst = u32x4{dec[0], dec[1], dec[2], dec[3]};
                *(u32x4 *)(dst + 16) = u32x4{dec[4], dec[5], dec[6], dec[7]};
            }
        }
        float *as_l = (float *)(st + A_BYTES + B_BYTES), *ws_l = (float *)(st + A_BYTES + B_BYTES + AS_BYTES);
#pragma unroll
        for (int i = 0; i < NAS; ++i)                            // blocks past the end of K: scale 0, no contribution
            if (tid + 256 * i < BM3 * KC) as_l[tid + 256 * i] = kb0 + (tid + 256 * i) % KC < KB ? ras[i] : 0.f;
#pragma unroll
        for (int i = 0; i < NWS; ++i) ws_l[tid + 256 * i] = kb0 + (tid + 256 * i) % KC < KB ? __half2float(rws[i]) : 0.f;
    };

    // K slices (grid z, few workgroups against a long K): slice z takes its share of the K steps and leaves raw sums in
    // `partial` [z][M][partial_ld] for gemm_i8_slices_kernel, which adds the slices in their order
    const int kt_per = (KT + (int)gridDim.z - 1) / (int)gridDim.z;
    const int kt_lo = (int)blockIdx.z * kt_per, kt_hi = min(KT, kt_lo + kt_per);
    if (partial) {
        partial += (size_t)blockIdx.z * M * partial_ld + (size_t)blockIdx.x * BN3;
        c = partial - n0;                                // column n0 + j of this tile -> partial column blockIdx.x * BN3 + j
        alpha = 1.f;
        beta = 0.f;
    }
    const size_t ldo = partial ? (size_t)partial_ld : ldc;
    const int n_hi = partial ? n0 + BN3 : N;            // (a partial tile is written whole: its padding columns are sums over clamped rows, never read)
    load_stage(kt_lo);
    store_stage(lds3, kt_lo);
    __syncthreads();
    for (int kt = kt_lo; kt < kt_hi; ++kt) {
        const unsigned char *st = lds3 + ((kt - kt_lo) & 1) * STAGE;
        const bool more = kt + 1 < kt_hi;
        if (more) load_stage(kt + 1);
        const float *as_l = (const float *)(st + A_BYTES + B_BYTES), *ws_l = (const float *)(st + A_BYTES + B_BYTES + AS_BYTES);
        float wsc[4][KCW];
#pragma unroll
        for (int ni = 0; ni < 4; ++ni) {
            if (SPLITK) {
#pragma unroll
                for (int jj = 0; jj < KCW; ++jj) wsc[ni][jj] = ws_l[(wn0 + ni * 16 + r) * KC + jw + 4 * jj];
            } else {
#pragma unroll
                for (int q = 0; q < KC / 4; ++q) {
                    const f32x4 v = *(const f32x4 *)(ws_l + (wn0 + ni * 16 + r) * KC + q * 4);
                    wsc[ni][q * 4 % KCW] = v.x; wsc[ni][(q * 4 + 1) % KCW] = v.y; wsc[ni][(q * 4 + 2) % KCW] = v.z; wsc[ni][(q * 4 + 3) % KCW] = v.w;
                }
            }
        }
        // (row tile, block) steps, software-pipelined: a step's dots are issued one at a time between the
        // rescales of the previous step's dots, so the matrix pipe runs under the vector work even with a
        // single wavefront on the SIMD. The empty asm statements fix that order for the compiler, which
        // otherwise issues every dot of the K step first and runs out of registers.
        i32x4 dprev[4];
        float asc[4][KCW];
#pragma unroll
        for (int t = 0; t <= WM * KCW; ++t) {
            const int mi = t / KCW, jj = t % KCW;
            const int pm = (t - 1) / KCW, pj = (t - 1) % KCW;
            i32x4 dcur[4];
            long a = 0;
            if (t < WM * KCW) a = *(const long *)(st + (wm0 + mi * 16 + r) * ROW + (jw + jstep * jj) * 32 + g * 8);
            if (t > 0 && pj == 0) {             // the previous row tile's activation scales
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (SPLITK) {
#pragma unroll
                        for (int q = 0; q < KCW; ++q) asc[i][q] = as_l[(wm0 + pm * 16 + g * 4 + i) * KC + jw + 4 * q];
                    } else {
#pragma unroll
                        for (int q = 0; q < KC / 4; ++q) {
                            const f32x4 v = *(const f32x4 *)(as_l + (wm0 + pm * 16 + g * 4 + i) * KC + q * 4);
                            asc[i][q * 4 % KCW] = v.x; asc[i][(q * 4 + 1) % KCW] = v.y; asc[i][(q * 4 + 2) % KCW] = v.z; asc[i][(q * 4 + 3) % KCW] = v.w;
                        }
                    }
                }
            }
#pragma unroll
            for (int ni = 0; ni < 4; ++ni) {
                if (t < WM * KCW) {
                    const long b = *(const long *)(st + A_BYTES + (wn0 + ni * 16 + r) * ROW + (jw + jstep * jj) * 32 + g * 8);
                    dcur[ni] = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b, i32x4{0, 0, 0, 0}, 0, 0, 0);
                }
                if (t > 0) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[pm][ni][i] += (float)dprev[ni][i] * (asc[i][pj] * wsc[ni][pj]);
                    asm volatile("" : "+v"(acc[pm][ni]));
                }
            }
#pragma unroll
            for (int ni = 0; ni < 4; ++ni) dprev[ni] = dcur[ni];
        }
        if (more) store_stage(lds3 + ((kt + 1 - kt_lo) & 1) * STAGE, kt + 1);
        __syncthreads();
    }

    if (SPLITK) {
        // partial sums of the four wavefronts -> LDS (the stages are free: the loop ended on a barrier), then
        // wavefront w adds column tile w in the fixed order 0,1,2,3 and writes it
        f32x4 *red = (f32x4 *)lds3;                      // [wave][mi][ni][lane]
#pragma unroll
        for (int mi = 0; mi < WM; ++mi)
#pragma unroll
            for (int ni = 0; ni < 4; ++ni) red[((wave * WM + mi) * 4 + ni) * 64 + lane] = acc[mi][ni];
        __syncthreads();
#pragma unroll
        for (int mi = 0; mi < WM; ++mi) {
            f32x4 sum = red[((0 * WM + mi) * 4 + wave) * 64 + lane];
#pragma unroll
            for (int w = 1; w < 4; ++w) sum += red[((w * WM + mi) * 4 + wave) * 64 + lane];
            const int col = n0 + wave * 16 + r;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = m0 + mi * 16 + g * 4 + i;
                if (row >= M || col >= n_hi) continue;
                float *dst = c + (size_t)row * ldo + col;
                const float v = alpha * sum[i];
                *dst = beta == 0.f ? v : v + beta * *dst;
            }
        }
        return;
    }
#pragma unroll
    for (int mi = 0; mi < WM; ++mi)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = m0 + wm0 + mi * 16 + g * 4 + i;
            if (row >= M) continue;
#pragma unroll
            for (int ni = 0; ni < 4; ++ni) {
                const int col = n0 + wn0 + ni * 16 + r;
                if (col >= n_hi) continue;
                float *dst = c + (size_t)row * ldo + col;
                const float v = alpha * acc[mi][ni][i];
                *dst = beta == 0.f ? v : v + beta * *dst;
            }
        }
}

// ------------------------------------------------------------------------------------ bf16 MFMA
constexpr int G2_TILE_K = 32;                                // k extent of a block of the tiled bf16 operands = the kernel's K step
__device__ __forceinline__ unsigned short bf16_rne(float x) {
    unsigned u = __float_as_uint(x);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
}

// The activation operand of the MFMA kernel is a bf16 copy made per call, laid out for its loads: 16 rows x 32 k (1 KiB) per
// block, blocks k-major within a group of 16 rows - [rows / 16][K / 32][16][32]. One LDS-writing load of a wavefront (16 rows
// x 64 bytes of one K step) is then 1 KiB of consecutive memory, eight whole 128-byte lines, where a row-major operand gives
// the L2 sixteen 64-byte requests, which it serves at the rate of 128-byte ones. Rows are padded to a multiple of 16 with zeros.
__device__ __forceinline__ size_t bf16_tiled_index(size_t row, size_t k0, size_t K) {
    return (((row >> 4) * (K / G2_TILE_K) + k0 / G2_TILE_K) * 16 + (row & 15)) * G2_TILE_K + (k0 % G2_TILE_K);
}

// device row layout -> bf16 tiled copy: value = code * f32(f16 scale), rounded to bf16
template <int DT>
__global__ void dequant_bf16_kernel(const uint8_t *__restrict__ qs, const __half *__restrict__ sc, unsigned short *__restrict__ out,
                                    size_t N, size_t K) {
    // one thread per 8 consecutive k of one row
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t per_row = K / 8, rows = (N + 15) & ~(size_t)15;
    if (i >= rows * per_row) return;
    const size_t n = i / per_row, k0 = (i % per_row) * 8;
    if (n >= N) {
        *(u32x4 *)(out + bf16_tiled_index(n, k0, K)) = u32x4{0u, 0u, 0u, 0u};
        return;
    }
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
    *(u32x4 *)(out + bf16_tiled_index(n, k0, K)) = o;
}

// A wavefront rounds one 1 KiB block of the tiled copy - 16 rows x 32 k: lane = 4 * row + part reads 8 consecutive floats of
// its row (the 16 rows' 128-byte lines, whole) and writes its 16 bytes of the block (1 KiB of consecutive memory); consecutive
// wavefronts take consecutive k blocks of the same 16 rows. VEC: the rows are 16-byte aligned and the loads are two dwordx4.
template <bool VEC>
__global__ __launch_bounds__(256) void act_bf16_kernel(const float *__restrict__ a, size_t lda, unsigned short *__restrict__ out, size_t M, size_t K) {
    const size_t wave = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63, row = lane >> 2, part = lane & 3;
    const size_t kblocks = K / G2_TILE_K, row_tiles = (M + 15) >> 4;
    if (wave >= row_tiles * kblocks) return;
    const size_t m = (wave / kblocks) * 16 + row, k0 = (wave % kblocks) * G2_TILE_K + part * 8;
    u32x4 o = u32x4{0u, 0u, 0u, 0u};                       // rows past M: zeros
    if (m < M) {
        const float *p = a + m * lda + k0;
        float v[8];
        if (VEC) {
            const f32x4 x = *(const f32x4 *)p, y = *(const f32x4 *)(p + 4);
            v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w; v[4] = y.x; v[5] = y.y; v[6] = y.z; v[7] = y.w;
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = p[i];
        }
        o.x = (unsigned)bf16_rne(v[0]) | ((unsigned)bf16_rne(v[1]) << 16);
        o.y = (unsigned)bf16_rne(v[2]) | ((unsigned)bf16_rne(v[3]) << 16);
        o.z = (unsigned)bf16_rne(v[4]) | ((unsigned)bf16_rne(v[5]) << 16);
        o.w = (unsigned)bf16_rne(v[6]) | ((unsigned)bf16_rne(v[7]) << 16);
    }
    *(u32x4 *)(out + bf16_tiled_index(m, k0, K)) = o;
}

// ---- wide-tile kernel: workgroup tile (WM*64) x 256, K step 32, v_mfma_f32_32x32x16_bf16.
// 2 x 2 wavefronts, each (WM*32) x (WN*32) outputs = WM x WN tiles of 32x32 (accumulators: WM*WN*16
// registers; WN = 4, or 3 for the narrower tiles of a last partial round). Operands go global -> LDS directly (global_load_lds_dwordx4: each wavefront load
// fills 1 KiB = 16 rows of 64 B, no staging registers, no LDS store instructions). Rows are not
// padded; the 16-byte chunk c of row r sits at slot c ^ ((r >> 2) & 3), chosen on the global side
// of the load, so that the 16 consecutive rows of a fragment read hit 16 distinct bank groups.
// Four LDS stages: the loads of K steps kt+1..kt+3 are in flight during the MFMAs of step kt - a
// load round trip through L2 under this traffic takes about as long as two K steps of MFMAs.
// The loads of a stage are issued in two parts, the weight rows with the first half of a K step's MFMAs and the
// activation rows with the second half, one load per MFMA: issued back to back, the four wavefronts' loads queue
// up in the CU's address unit and the wavefronts stall there with their MFMAs behind them (measured: 3-5 %).
// The wavefront waits on its own loads by count (s_waitcnt vmcnt) and the stages are handed over
// with a bare s_barrier: a fence would drain the younger stages' loads as well.
// Tile order: workgroup ids go round-robin over the 8 XCDs, so id -> (xcd, slot) -> a contiguous
// run of tiles per XCD, M fastest: the workgroups that share a weight column tile run on one L2.
constexpr int G2_BK = 32, G2_ROW = 64, G2_BN = 256;
static_assert(G2_BK == G2_TILE_K, "a block of the tiled operands is one K step");
using f32x16 = __attribute__((ext_vector_type(16))) float;


// Instruction order of half a K step: two MFMAs first (the wait in front of them then covers only reads issued long
// ago), then every LDS read of the next fragment with an MFMA behind it (so that they are back when the next half
// starts), then the V global->LDS loads one per MFMA. The address unit of a CU takes about 16 cycles per 16-byte
// wavefront load; four wavefronts issuing theirs back to back stall on its queue, with an MFMA between two loads they do not.
template <int NMMA, int NFR, int V>
__device__ __forceinline__ void sched_half() {
    constexpr int REST = NMMA - 2 - NFR;                     // MFMAs left once the reads are placed
    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
#pragma unroll
    for (int i = 0; i < NFR; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        if (REST <= 0 ? i < V : i >= NFR - (V - REST) ) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // loads that find no MFMA of their own
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
    if constexpr (REST > 0) {
#pragma unroll
        for (int i = 0; i < (V < REST ? V : REST); ++i) {
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        if constexpr (REST > V) __builtin_amdgcn_sched_group_barrier(0x008, REST - V, 0);
    }
}

// The weight operand of the bf16 kernel, dequantized while it is staged (as aion's GPU GEMM does, backend/gpu/kernels/
// matmul_q8_mx16.wgsl): thread t of the workgroup owns column n0 + t of the tile. Every four K steps it requests the next
// four quant blocks of its row (64 bytes of q4 codes, 128 of q8, and their four f16 scales) into registers - three such
// groups rotate: one being converted, one waiting, one in flight - and in every K step it converts one block to 32 bf16
// values (code * f32(scale), rounded to nearest even: the bits a separate dequantization pass would give) and writes
// them as the 64-byte row of the LDS stage two K steps ahead, in the swizzled chunk order the fragment reads expect.
// The L2 then delivers 18 or 34 bytes per 32 weights instead of 64, and no bf16 copy of the weight exists.
template <int BDT>
struct WGroup {
    static constexpr int NQ = BDT == AIONHIP_Q8_0 ? 8 : 4;      // 16-byte loads per group of four blocks
    u32x4 q[NQ];
    unsigned short s[4];
};
template <int BDT>
struct WSource {
    const uint8_t *row;          // this thread's weight row (codes)
    const __half *sc;            // its block scales
    int kb;                      // blocks per row
    // load i of a group request (i < NQ: 16 bytes of codes, then the four scales), for callers that space the loads out
    __device__ __forceinline__ void request_one(int group, WGroup<BDT> &g, int i) const {
        constexpr int PER = BDT == AIONHIP_Q8_0 ? 2 : 1;
        constexpr int NQ = WGroup<BDT>::NQ;
        if (i < NQ) {
            const int b = min(group * 4 + i / PER, kb - 1);
            g.q[i] = *(const u32x4 *)(row + (size_t)b * (16 * PER) + (i % PER) * 16);
        } else {
            const int b = min(group * 4 + (i - NQ), kb - 1);
            g.s[i - NQ] = __half_as_ushort(sc[b]);
        }
    }
    __device__ __forceinline__ void request(int group, WGroup<BDT> &g) const {
        constexpr int PER = BDT == AIONHIP_Q8_0 ? 2 : 1;        // 16-byte chunks per block
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int b = min(group * 4 + j, kb - 1);            // past the end: a harmless repeat into a dead stage
#pragma unroll
            for (int h = 0; h < PER; ++h) g.q[j * PER + h] = *(const u32x4 *)(row + (size_t)b * (16 * PER) + h * 16);
            g.s[j] = __half_as_ushort(sc[b]);
        }
    }
};
// block j of a group -> 32 bf16 values into the 64-byte stage row `dst` of a thread whose row swizzle is `swz`
// Conversion state of one block, advanced element by element so that the caller can put one element's three vector
// instructions behind each MFMA: element e (0 .. 31) of block j of a group; after the eighth element of a 16-byte chunk the
// chunk is written to the stage row.
template <int BDT>
struct DeqBlock {
    float sc, off;
    unsigned lo, hi;
    float f[8];
    template <int J, int E>
    __device__ __forceinline__ void element(const WGroup<BDT> &g, unsigned char *dst, int swz) {
        using f32x2_t = __attribute__((ext_vector_type(2))) float;
        using bf16x2_t = __attribute__((ext_vector_type(2))) __bf16;
        auto pk = [](float a, float b) { return __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2_t{a, b}, bf16x2_t)); };
        constexpr int d = E / 8, i = E % 8;
        if constexpr (E == 0 || E == 16) {
            sc = __half2float(__ushort_as_half(g.s[J]));
            off = (BDT == AIONHIP_Q4_0 ? -8.f : -128.f) * sc;     // (c - 8) * s = fma(c, s, -8 s): one rounding, the same value
        }
        if constexpr (i == 0) {
            if constexpr (BDT == AIONHIP_Q4_0) {
                // byte i of a word = e[8d + i] | e[8d + 4 + i] << 4
                const unsigned w = d == 0 ? g.q[J].x : d == 1 ? g.q[J].y : d == 2 ? g.q[J].z : g.q[J].w;
                lo = w & 0x0F0F0F0Fu;
                hi = (w >> 4) & 0x0F0F0F0Fu;
            } else {
                // signed code c = u - 128 with u = c ^ 0x80
                const u32x4 w = g.q[J * 2 + (d >> 1)];
                lo = ((d & 1) ? w.z : w.x) ^ 0x80808080u;
                hi = ((d & 1) ? w.w : w.y) ^ 0x80808080u;
            }
        }
        f[i] = fmaf((float)(((i < 4 ? lo : hi) >> (8 * (i & 3))) & 0xFFu), sc, off);
        if constexpr (i == 7) *(u32x4 *)(dst + ((d ^ swz) * 16)) = u32x4{pk(f[0], f[1]), pk(f[2], f[3]), pk(f[4], f[5]), pk(f[6], f[7])};
    }
};
template <int I, int E, class F>
__device__ __forceinline__ void static_for_gemm(F &&f) {
    if constexpr (I < E) {
        f(std::integral_constant<int, I>{});
        static_for_gemm<I + 1, E>(f);
    }
}
constexpr int vmcnt_lgkm0_imm(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4); }   // vmcnt <= n and lgkmcnt == 0

// one workgroup tile: rows m0 .., columns n0 .. of C (N is the column bound of W and C as passed)
// BDT = 0: W is a bf16 copy in the tiled layout; BDT = a block format: the weight itself (wq, wsc), dequantized while staged
template <int WM, int NST, int WN, int BDT = 0>
__device__ __forceinline__ void gemm_bf16_tile(unsigned char *lds2, const unsigned short *__restrict__ A, const unsigned short *__restrict__ W,
                                               float *__restrict__ c, int M, int N, int K, size_t ldc, float alpha, float beta, int m0, int n0,
                                               const uint8_t *__restrict__ wq = nullptr, const __half *__restrict__ wsc = nullptr) {
    static_assert(BDT == 0 || NST == 4, "the dequantizing form writes the stage two K steps ahead of a four-stage ring");
    constexpr int BM2 = WM * 64;
    constexpr int BN2 = WN * 64;                             // 256 columns, or 192 for the last partial round of tiles
    constexpr int A_BYTES = BM2 * G2_ROW, B_BYTES = BN2 * G2_ROW, STAGE = A_BYTES + B_BYTES;
    constexpr int NA = WM, NB = WN;                          // wavefront loads (16 rows each) per stage
    constexpr int NL = NA + NB;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l31 = lane & 31, lh = lane >> 5;
    const int wrow = (wave >> 1) * (WM * 32), wcol = (wave & 1) * (WN * 32);

    f32x16 acc[WM][WN];
#pragma unroll
    for (int mi = 0; mi < WM; ++mi)
#pragma unroll
        for (int ni = 0; ni < WN; ++ni)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mi][ni][i] = 0.f;

    // load i of this wavefront covers tile rows i*64 + wave*16 .. +16; lane -> (row lane>>2, slot lane&3)
    // (operands in the tiled layout: the wavefront's 16 rows of a K step are one 1 KiB block; within it lane -> row
    // lane >> 2, chunk (lane & 3) ^ ((lane >> 4) & 3), the swizzle the fragment reads undo)
    const int KT = K / G2_BK;
    const int in_block = (lane >> 2) * G2_BK + (((lane & 3) ^ ((lane >> 4) & 3)) * 8);
    const int a_blocks = (M + 15) >> 4, w_blocks = (N + 15) >> 4;
    const unsigned short *ga[NA], *gb[NB];
#pragma unroll
    for (int i = 0; i < NA; ++i) ga[i] = A + (size_t)min((m0 >> 4) + i * 4 + wave, a_blocks - 1) * KT * (16 * G2_BK) + in_block;
#pragma unroll
    for (int i = 0; i < NB; ++i) gb[i] = BDT ? nullptr : W + (size_t)min((n0 >> 4) + i * 4 + wave, w_blocks - 1) * KT * (16 * G2_BK) + in_block;
    (void)w_blocks;
    // dequantizing form: this thread's weight row and its stage row
    WSource<BDT ? BDT : AIONHIP_Q4_0> wsrc{};
    WGroup<BDT ? BDT : AIONHIP_Q4_0> g_cur, g_nxt, g_fut;
    const int b_row = min(tid, BN2 - 1), b_swz = (b_row >> 2) & 3;
    if constexpr (BDT != 0) {
        const size_t n = (size_t)min(n0 + b_row, N - 1);
        wsrc.row = wq + n * (BDT == AIONHIP_Q8_0 ? (size_t)K : (size_t)K / 2);
        wsrc.sc = wsc + n * (size_t)(K / 32);
        wsrc.kb = K / 32;
    }
    unsigned char *const b_stage_row = lds2 + A_BYTES + b_row * G2_ROW;       // this thread's row in stage 0
    using BT = std::integral_constant<int, BDT ? BDT : AIONHIP_Q4_0>;
    DeqBlock<BT::value> dq;
    auto deq_whole = [&](const WGroup<BT::value> &g, auto jc, int kt) __attribute__((always_inline)) {
        constexpr int J = decltype(jc)::value;
        if (tid < BN2) {
            unsigned char *dst = b_stage_row + (kt % NST) * STAGE;
            static_for_gemm<0, 32>([&](auto ec) __attribute__((always_inline)) { dq.template element<J, decltype(ec)::value>(g, dst, b_swz); });
        }
    };

    auto issue_loads = [&](int kt, bool a_part, bool b_part) {
#if defined(__HIP_DEVICE_COMPILE__)   // the builtin exists in the device pass only
        unsigned char *stage = lds2 + (kt % NST) * STAGE + wave * 16 * G2_ROW;
        const size_t k = (size_t)min(kt, KT - 1) * (16 * G2_BK);   // the next block of the row group; past the end: a harmless repeat into a dead stage
        if (a_part)
#pragma unroll
            for (int i = 0; i < NA; ++i)
                __builtin_amdgcn_global_load_lds(ga[i] + k, (lds_void *)(stage + i * 64 * G2_ROW), 16, 0, 0);
        if (b_part && BDT == 0)
#pragma unroll
            for (int i = 0; i < NB; ++i)
                __builtin_amdgcn_global_load_lds(gb[i] + k, (lds_void *)(stage + A_BYTES + i * 64 * G2_ROW), 16, 0, 0);
#endif
    };

    auto issue_a_load = [&](int kt, int i) {
#if defined(__HIP_DEVICE_COMPILE__)
        unsigned char *stage = lds2 + (kt % NST) * STAGE + wave * 16 * G2_ROW;
        const size_t k = (size_t)min(kt, KT - 1) * (16 * G2_BK);
        __builtin_amdgcn_global_load_lds(ga[i] + k, (lds_void *)(stage + i * 64 * G2_ROW), 16, 0, 0);
#endif
    };
    (void)issue_a_load;

    // fragment of sub-step ks: row (base + l31), chunk ks*2 + lh, at slot chunk ^ ((l31 >> 2) & 3)
    const int swz = (l31 >> 2) & 3;
    int foff[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) foff[ks] = l31 * G2_ROW + (((ks * 2 + lh) ^ swz) * 16);
    const int fa = wrow * G2_ROW, fb = A_BYTES + wcol * G2_ROW;

    struct Frag {
        u32x4 a[WM], b[WN];
    };
    auto read_frag = [&](Frag &f, int kt, int ks) {
        const unsigned char *st = lds2 + (kt % NST) * STAGE;
#pragma unroll
        for (int ni = 0; ni < WN; ++ni) f.b[ni] = *(const u32x4 *)(st + fb + ni * 32 * G2_ROW + foff[ks]);
#pragma unroll
        for (int mi = 0; mi < WM; ++mi) f.a[mi] = *(const u32x4 *)(st + fa + mi * 32 * G2_ROW + foff[ks]);
    };
    auto mma = [&](const Frag &f) {
#pragma unroll
        for (int mi = 0; mi < WM; ++mi)
#pragma unroll
            for (int ni = 0; ni < WN; ++ni)
                acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, f.b[ni]), __builtin_bit_cast(bf16x8, f.a[mi]), acc[mi][ni], 0, 0, 0);
    };
    constexpr int NMMA = WM * WN, NFR = WM + WN;

    Frag f0, f1;
    if constexpr (BDT == 0) {
    // issue order: A0 B0 A1 B1 .. A(NST-2) | K step 0: B(NST-2), A(NST-1) | K step 1: B(NST-1), A(NST) | ...
#pragma unroll
    for (int i = 0; i < NST - 2; ++i) issue_loads(i, true, true);
    issue_loads(NST - 2, true, false);
    __builtin_amdgcn_s_waitcnt(vmcnt_imm((NST - 3) * NL + NA));   // stage 0 of this wavefront has landed
    __builtin_amdgcn_s_barrier();                            // ... and everybody else's
    read_frag(f0, 0, 0);
    for (int kt = 0; kt < KT; ++kt) {
        // sub-step 0 while the fragments of sub-step 1 are read
        read_frag(f1, kt, 1);
        issue_loads(kt + NST - 2, false, true);
        mma(f0);
        if constexpr (WM >= 2) sched_half<NMMA, NFR, NB>();
        // stage kt+1 landed (stage kt+2 may still be in flight); past this barrier nobody reads stage kt-1
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((NST - 3) * NL));
        __builtin_amdgcn_s_barrier();
        // sub-step 1 while fragments 0 of the next K step are read, then the loads of stage kt+3
        // (an LDS-writing load may not move above an LDS read: reads first)
        read_frag(f0, kt + 1, 0);
        issue_loads(kt + NST - 1, true, false);
        mma(f1);
        if constexpr (WM >= 2) sched_half<NMMA, NFR, NA>();
    }
    } else {
    // Dequantizing form. Load order: groups 0 and 1 of the weight row, A0 A1 A2 | K step kt: (first of four: group kt/4 + 2),
    // A(kt+3). The weight block of K step kt + 2 is converted into its stage during the first half of K step kt.
    constexpr int NF = WGroup<BDT ? BDT : AIONHIP_Q4_0>::NQ + 4;  // loads of one group request
    wsrc.request(0, g_cur);
    wsrc.request(1, g_nxt);
#pragma unroll
    for (int i = 0; i < NST - 1; ++i) issue_loads(i, true, false);
    deq_whole(g_cur, std::integral_constant<int, 0>{}, 0);
    deq_whole(g_cur, std::integral_constant<int, 1>{}, 1);
    __builtin_amdgcn_s_waitcnt(vmcnt_lgkm0_imm((NST - 2) * NA));  // A of stage 0 has landed, the two converted blocks are written
    __builtin_amdgcn_s_barrier();
    read_frag(f0, 0, 0);
    // Half a K step: behind every MFMA one slice of everything else the half has to issue - the conversion of 16 / NMMA
    // weight elements (the matrix pipe takes 32 cycles per MFMA, the vector pipe 4 per instruction, and a wavefront issues
    // in order: what is to run in an MFMA's shadow has to stand behind it in the program), in the second half also one of
    // the global loads - pinned with scheduling barriers.
    auto half = [&](const Frag &f, int kt, auto jc, auto hc) __attribute__((always_inline)) {
        constexpr int j = decltype(jc)::value, hf = decltype(hc)::value;
        constexpr int J = j < 2 ? j + 2 : j - 2;                  // block of the group: 2, 3 of the current one, then 0, 1 of the next
        const WGroup<BT::value> &g = j < 2 ? g_cur : g_nxt;
        unsigned char *dst = b_stage_row + ((kt + 2) % NST) * STAGE;
        constexpr int NLD = hf == 1 ? NA + (j == 0 ? NF : 0) : 0; // global loads of this half
        static_for_gemm<0, NMMA>([&](auto ic) __attribute__((always_inline)) {
            constexpr int i = decltype(ic)::value, mi = i / WN, ni = i % WN;
            acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, f.b[ni]), __builtin_bit_cast(bf16x8, f.a[mi]), acc[mi][ni], 0, 0, 0);
            constexpr int e0 = hf * 16 + i * 16 / NMMA, e1 = hf * 16 + (i + 1) * 16 / NMMA;
            if (tid < BN2) static_for_gemm<e0, e1>([&](auto ec) __attribute__((always_inline)) { dq.template element<J, decltype(ec)::value>(g, dst, b_swz); });
            // loads: spread over the MFMAs (as many per MFMA as it takes)
            constexpr int l0 = i * NLD / NMMA, l1 = (i + 1) * NLD / NMMA;
            static_for_gemm<l0, l1>([&](auto lc) __attribute__((always_inline)) {
                constexpr int li = decltype(lc)::value;
                if constexpr (li < NA) issue_a_load(kt + NST - 1, li);
                else wsrc.request_one(kt / 4 + 2, g_fut, li - NA);
            });
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    auto step = [&](int kt, auto jc) __attribute__((always_inline)) {
        constexpr int j = decltype(jc)::value;
        read_frag(f1, kt, 1);
        __builtin_amdgcn_sched_barrier(0);
        half(f0, kt, jc, std::integral_constant<int, 0>{});
        // A of stage kt+1 landed (what was requested after it may still be in flight); the chunks converted so far are
        // written; past this barrier nobody reads stage kt-1
        __builtin_amdgcn_s_waitcnt(vmcnt_lgkm0_imm(j == 1 || j == 2 ? NA + NF : NA));
        __builtin_amdgcn_s_barrier();
        read_frag(f0, kt + 1, 0);
        __builtin_amdgcn_sched_barrier(0);
        // ... and the other half of the block (written before the barrier of the next K step, behind which stage kt+2 is first read)
        half(f1, kt, jc, std::integral_constant<int, 1>{});
    };
    for (int kt0 = 0; kt0 < KT; kt0 += 4) {
        step(kt0, std::integral_constant<int, 0>{});
        if (kt0 + 1 < KT) step(kt0 + 1, std::integral_constant<int, 1>{});
        if (kt0 + 2 < KT) step(kt0 + 2, std::integral_constant<int, 2>{});
        if (kt0 + 3 < KT) step(kt0 + 3, std::integral_constant<int, 3>{});
        g_cur = g_nxt;
        g_nxt = g_fut;
    }
    }
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));                // no LDS-writing load may outlive the workgroup

    // The products are taken transposed (weight fragment as the first operand): element i of lane l then belongs to output
    // row l % 32 (a token) and column (i / 4) * 8 + (l / 32) * 4 + i % 4, so every four accumulator elements are four
    // consecutive floats of a C row - 16-byte stores, a quarter of the store instructions of a lane-per-column layout.
    const bool vec_ok = (((uintptr_t)c | (ldc * sizeof(float))) & 15) == 0;
#pragma unroll
    for (int mi = 0; mi < WM; ++mi) {
        const int row = m0 + wrow + mi * 32 + l31;
        if (row >= M) continue;
        float *crow = c + (size_t)row * ldc;
#pragma unroll
        for (int ni = 0; ni < WN; ++ni)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int col = n0 + wcol + ni * 32 + g * 8 + lh * 4;
                if (col >= N) continue;
                f32x4 v = f32x4{acc[mi][ni][g * 4], acc[mi][ni][g * 4 + 1], acc[mi][ni][g * 4 + 2], acc[mi][ni][g * 4 + 3]} * alpha;
                if (vec_ok && col + 3 < N) {
                    if (beta != 0.f) v += *(const f32x4 *)(crow + col) * beta;
                    *(f32x4 *)(crow + col) = v;
                } else {
                    const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        if (col + t < N) crow[col + t] = beta == 0.f ? e[t] : e[t] + beta * crow[col + t];
                }
            }
    }
}

template <int WM, int NST, int WN, int BDT>
__global__ __launch_bounds__(256) void gemm_bf16_wide_kernel(const unsigned short *__restrict__ A, const uint8_t *__restrict__ wq, const __half *__restrict__ wsc,
                                                             float *__restrict__ c, int M, int N, int K, size_t ldc, float alpha,
                                                             float beta, int tiles_m, int tiles) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds2[];
    const int per_xcd = (int)gridDim.x >> 3;
    const int t = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
    if (t >= tiles) return;
    // (BDT = 0: wq is the weight's bf16 copy in the tiled layout)
    gemm_bf16_tile<WM, NST, WN, BDT>(lds2, A, (const unsigned short *)wq, c, M, N, K, ldc, alpha, beta, (t % tiles_m) * (WM * 64), (t / tiles_m) * (WN * 64), wq, wsc);
}

// 256-row tiles over N = tw * 256 + (a rest covered by tn tiles of 192 columns), ONE launch: the column tiles go
// wide, wide, narrow, narrow, ... while both kinds last. A CU's first tile is then wide on half of the CUs and narrow on the
// other half, the CUs that finish early pick up wide tiles next, and the epilogues (64 MB of f32 stores that would otherwise
// hit the HBM from every CU at the same moment, with the matrix pipes idle) fall into the others' main loops.
template <int NST, int BDT>
__global__ __launch_bounds__(256) void gemm_bf16_mixed_kernel(const unsigned short *__restrict__ A, const uint8_t *__restrict__ wq, const __half *__restrict__ wsc,
                                                              float *__restrict__ c, int M, int N, int K, size_t ldc, float alpha,
                                                              float beta, int tiles_m, int tw, int tn) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds2[];
    const int per_xcd = (int)gridDim.x >> 3;
    const int t = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
    if (t >= tiles_m * (tw + tn)) return;
    const int cg = t / tiles_m, m0 = (t % tiles_m) * 256;
    const int fb = min(tw, tn) >> 1;                         // whole blocks of wide, wide, narrow, narrow
    bool wide;
    int idx;
    if (cg < 4 * fb) {
        wide = (cg & 3) < 2;
        idx = (cg >> 2) * 2 + (cg & 1);
    } else {
        const int rest = cg - 4 * fb, rest_wide = tw - 2 * fb;
        wide = rest < rest_wide;
        idx = 2 * fb + (wide ? rest : rest - rest_wide);
    }
    if (wide) gemm_bf16_tile<4, NST, 4, BDT>(lds2, A, (const unsigned short *)wq, c, M, N, K, ldc, alpha, beta, m0, idx * 256, wq, wsc);
    else gemm_bf16_tile<4, NST, 3, BDT>(lds2, A, (const unsigned short *)wq, c, M, N, K, ldc, alpha, beta, m0, tw * 256 + idx * 192, wq, wsc);
}

// Tile choice by a small cost model fitted to measurements on one MI355X (q4, K = 2048..8192, 24..2048
// rows): a lone workgroup of each shape costs `us_per_block` per quant block of K; workgroups beyond one
// per CU overlap by the factor `overlap` (two resident per CU hide each other's staging).
struct GiShape { int wm; bool split; float us_per_block, overlap; };
constexpr GiShape GI_SHAPES[6] = {
    {4, false, 0.81f, 1.40f}, {2, false, 0.44f, 1.25f}, {1, false, 0.284f, 1.55f},
    {4, true, 0.253f, 1.45f}, {2, true, 0.164f, 1.50f}, {1, true, 0.121f, 1.85f},
};
// The K slices of gemm_i8_lds_kernel folded in slice order: C = alpha * (p[0] + p[1] + ...) + beta * C, one thread per
// (row, four columns of a tile).
__global__ __launch_bounds__(256) void gemm_i8_slices_kernel(GemmSegs segs, const float *__restrict__ partial, int M, int slices, int partial_ld,
                                                             int bn, float alpha, float beta) {
    const int quads = partial_ld >> 2;
    const size_t id = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= (size_t)M * quads) return;
    const int row = (int)(id / quads), pc = (int)(id % quads) * 4, tile = pc / bn;
    int si = 0;
#pragma unroll
    for (int i = 1; i < 4; ++i)
        if (i < segs.count && tile >= segs.first_tile[i]) si = i;
    const int col = pc - segs.first_tile[si] * bn;
    if (col >= segs.n[si]) return;
    f32x4 sum = *(const f32x4 *)(partial + (size_t)row * partial_ld + pc);
    for (int z = 1; z < slices; ++z) sum += *(const f32x4 *)(partial + ((size_t)z * M + row) * partial_ld + pc);
    float *dst = segs.c[si] + (size_t)row * segs.ldc[si] + col;
    const float e[4] = {sum.x, sum.y, sum.z, sum.w};
#pragma unroll
    for (int t = 0; t < 4; ++t)
        if (col + t < segs.n[si]) dst[t] = beta == 0.f ? alpha * e[t] : alpha * e[t] + beta * dst[t];
}

// How many K slices a launch of `wgs` workgroups (each able to overlap `overlap` to a CU, `us_per_block` per quant block of a
// lone one) over `kt` K steps of `blocks` quant blocks is cut into. Slices pay when the modelled time with them, the
// launch that adds them up included, is under three quarters of the time without (measured: 4096 x 14336 at 16 rows
// 52 -> 22 us in 7 slices, 2048 x 8192 33 -> 15 us, 4096 x 4096 20 -> 15 us; K = 2048 never: the second launch costs what
// the slices save).
inline int i8_k_slices(const aionhip_ctx *ctx, float wgs, float overlap, int kt, float us_per_block, float blocks) {
    const float cus = (float)(ctx->cu_count > 0 ? ctx->cu_count : 256);
    const float rounds = wgs / (cus * overlap);
    if (ctx->no_scratch_paths || rounds >= 0.75f || kt < 8) return 1;
    int s = (int)(1.f / rounds + 0.5f);
    s = s < kt / 4 ? s : kt / 4;                          // at least four K steps per slice
    s = s > 8 ? 8 : s;
    if (s < 2) return 1;
    const float alone = us_per_block * blocks;
    const float sliced = alone / (float)s * (rounds * (float)s > 1.f ? rounds * (float)s : 1.f) + 4.f;
    return sliced < 0.75f * alone ? s : 1;
}

template <int DT, int WM, int KC, bool SPLITK>
int launch_i8_lds(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, size_t m, PreparedAct act,
                  float alpha, float beta) {
    constexpr int BM3 = (SPLITK ? 16 : 32) * WM, BN3 = SPLITK ? 64 : 128;
    constexpr int LDS = 2 * ((BM3 + BN3) * GiCfg<KC>::ROW + (BM3 + BN3) * KC * 4);
    static_assert(LDS <= 160 * 1024, "two stages must fit the CU's LDS");
    static_assert(!SPLITK || 4 * WM * 4 * 64 * 16 <= LDS, "the split-K reduction reuses the stages");
    static bool attr = false;
    if (!attr) {
        HIP_TRY(ctx, hipFuncSetAttribute((const void *)gemm_i8_lds_kernel<DT, WM, KC, SPLITK>, hipFuncAttributeMaxDynamicSharedMemorySize, LDS));
        attr = true;
    }
    GemmSegs segs{};
    segs.count = count;
    int tiles = 0;
    for (int i = 0; i < count; ++i) {
        segs.qs[i] = ws[i]->qs;
        segs.sc[i] = ws[i]->sc;
        segs.c[i] = cs[i];
        segs.ldc[i] = ldcs[i];
        segs.n[i] = (int)ws[i]->n;
        segs.first_tile[i] = tiles;
        tiles += (int)((ws[i]->n + BN3 - 1) / BN3);
    }
    const int m_tiles = (int)((m + BM3 - 1) / BM3), kt = (int)(((ws[0]->k >> 5) + KC - 1) / KC);
    // Few workgroups against a long K (a short prompt or a batch of 9..64 rows on a narrow weight): the K steps are cut into
    // slices across more workgroups and a second, small launch adds the slices in order - the same sums in the same
    // order per slice, the slices in a fixed order, so the result does not depend on timing.
    constexpr GiShape SHAPE = GI_SHAPES[(SPLITK ? 3 : 0) + (WM == 4 ? 0 : WM == 2 ? 1 : 2)];
    static_assert(SHAPE.wm == WM && SHAPE.split == SPLITK, "shape table order");
    int slices = i8_k_slices(ctx, (float)tiles * (float)m_tiles, SHAPE.overlap, kt, SHAPE.us_per_block, (float)(ws[0]->k >> 5));
    while (slices > 1 && (kt + slices - 1) / slices * (slices - 1) >= kt) --slices;      // no empty slice
    float *partial = nullptr;
    const int partial_ld = tiles * BN3;
    if (slices > 1) {
        const int rc = ensure_scratch2(ctx, (size_t)slices * m * partial_ld * sizeof(float));
        if (rc) return rc;
        partial = (float *)ctx->scratch2;
    }
    const dim3 grid((unsigned)tiles, (unsigned)m_tiles, (unsigned)slices);
    launch_k(ctx, gemm_i8_lds_kernel<DT, WM, KC, SPLITK>, grid, dim3(256), LDS, segs, act.q, act.scale, (int)m, (int)ws[0]->k, alpha, beta, partial, partial_ld);
    if (slices > 1) {
        const size_t threads = m * (size_t)(partial_ld >> 2);
        launch_k(ctx, gemm_i8_slices_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, segs, partial, (int)m, slices, partial_ld, BN3, alpha, beta);
    }
    return AIONHIP_OK;
}

// the cheapest shape for m rows against an n x k weight and its modelled time per quant block of K
int pick_i8_shape(const aionhip_ctx *ctx, size_t m, size_t n, size_t k, float *us_per_block) {
    const float cus = (float)(ctx->cu_count > 0 ? ctx->cu_count : 256);
    int best = 0;
    float best_t = 0.f;
    for (int i = 0; i < 6; ++i) {
        const GiShape &g = GI_SHAPES[i];
        if (g.split && k < 256) continue;                // a split-K step is 8 blocks
        const size_t bm = (size_t)(g.split ? 16 : 32) * g.wm, bn = g.split ? 64 : 128;
        const float wgs = (float)(((m + bm - 1) / bm) * ((n + bn - 1) / bn));
        const float rounds = wgs / (cus * g.overlap);
        const float t = g.us_per_block * (rounds > 1.f ? rounds : 1.f);
        if (i == 0 || t < best_t) { best = i; best_t = t; }
    }
    if (us_per_block) *us_per_block = best_t;
    return best;
}
// the tile shape is chosen for the columns of all the weights together (their tiles share the launch)
template <int DT>
int launch_i8_lds_pick(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, size_t m,
                       PreparedAct act, float alpha, float beta) {
    size_t n_total = 0;
    for (int i = 0; i < count; ++i) n_total += ws[i]->n;
    const int best = pick_i8_shape(ctx, m, n_total, ws[0]->k, nullptr);
    switch (best) {
    case 0: return launch_i8_lds<DT, 4, 4, false>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
    case 1: return launch_i8_lds<DT, 2, 4, false>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
    case 2: return launch_i8_lds<DT, 1, 4, false>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
    case 3: return launch_i8_lds<DT, 4, 8, true>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
    case 4: return launch_i8_lds<DT, 2, 8, true>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
    default: return launch_i8_lds<DT, 1, 8, true>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
    }
}

}  // namespace

// In bf16 mode: is the bf16 MFMA kernel expected to beat the exact kernel for this shape? Up to a few hundred rows it
// is not - it streams a 2-byte copy of every weight (3.5x the q4 bytes), its 256-column tiles leave most CUs idle and
// one workgroup's K loop is a latency chain - and the exact kernel is then both the faster and the exact one.
// Modelled times in microseconds, constants fitted to a sweep of 9..512 rows over four weight shapes.
bool gemm_bf16_pays(const aionhip_ctx *ctx, size_t m, size_t n, size_t k) {
    float per_block = 0.f;
    const GiShape &g = GI_SHAPES[pick_i8_shape(ctx, m, n, k, &per_block)];
    const float blocks = (float)(k / 32);
    // (the exact kernel cuts a long K into slices across workgroups when its grid is sparse)
    const size_t bm = (size_t)(g.split ? 16 : 32) * g.wm, bn = g.split ? 64 : 128;
    const float wgs = (float)(((m + bm - 1) / bm) * ((n + bn - 1) / bn));
    const int kc = g.split ? 8 : 4;                      // (the launcher's KC per shape)
    const int slices = i8_k_slices(ctx, wgs, g.overlap, (int)((k / 32 + kc - 1) / kc), g.us_per_block, blocks);
    const float cus = (float)(ctx->cu_count > 0 ? ctx->cu_count : 256);
    const float rounds = wgs * (float)slices / (cus * g.overlap);
    const float kernel_us = slices > 1 ? g.us_per_block * blocks / (float)slices * (rounds > 1.f ? rounds : 1.f) + 4.f : per_block * blocks;
    const float exact_us = kernel_us + 5.f + (float)m * (float)k * 4.f / 2.0e6f;               // + the int8 preparation of A
    // (constants fitted to both kernels' times over six weight shapes x 65..1024 rows, q4: the choice costs 0.3 % over
    // always taking the faster one; always exact would cost 36 %, always bf16 17 %)
    const float copy_us = (float)n * (float)k * 2.f / 3.0e6f;                                  // weight bytes at ~3 TB/s
    const float flop_us = 2.f * (float)m * (float)n * (float)k / 9.0e8f;                        // ~900 TFLOP/s
    const float chain_us = blocks * 0.24f;                                                       // one workgroup's K loop
    const float act_us = (float)m * (float)k * 6.f / 4.0e6f;                                     // the bf16 rounding of A
    const float bf16_us = fmaxf(fmaxf(copy_us, flop_us), chain_us) + act_us;
    return bf16_us < exact_us;
}

int launch_gemm_i8_few_rows(aionhip_ctx *ctx, const aionhip_weight *w, size_t m, PreparedAct act, float *c, size_t ldc, float alpha, float beta) {
    return w->dtype == AIONHIP_Q8_0 ? launch_i8_lds_pick<AIONHIP_Q8_0>(ctx, &w, &c, &ldc, 1, m, act, alpha, beta)
                                    : launch_i8_lds_pick<AIONHIP_Q4_0>(ctx, &w, &c, &ldc, 1, m, act, alpha, beta);
}

// 1..4 weights of one dtype, layout and K against the same prepared rows, one launch
int launch_gemm_i8_batch(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, size_t m,
                         PreparedAct act, float alpha, float beta) {
    if (count < 1 || count > 4) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "gemm: %d weights in one launch (1..4)", count);
    const char *name = ws[0]->dtype == AIONHIP_Q8_0 ? "gemm_i8_q8" : "gemm_i8_q4";
    ProfScope scope(ctx, name);
    const int rc = ws[0]->dtype == AIONHIP_Q8_0 ? launch_i8_lds_pick<AIONHIP_Q8_0>(ctx, ws, cs, ldcs, count, m, act, alpha, beta)
                                                 : launch_i8_lds_pick<AIONHIP_Q4_0>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
    if (rc) return rc;
    LAUNCH_CHECK(ctx, name);
    return AIONHIP_OK;
}

int launch_gemm_i8(aionhip_ctx *ctx, const aionhip_weight *w, size_t m, PreparedAct act, float *c, size_t ldc, float alpha, float beta) {
    const char *name = w->dtype == AIONHIP_Q8_0 ? "gemm_i8_q8" : "gemm_i8_q4";
    ProfScope scope(ctx, name);
    const int rc = launch_gemm_i8_few_rows(ctx, w, m, act, c, ldc, alpha, beta);
    if (rc) return rc;
    LAUNCH_CHECK(ctx, name);
    return AIONHIP_OK;
}

// The context's bf16 copy of a weight (tiled layout), built on first use: see aionhip_set_bf16_weight_copies.
static int bf16_copy_of(aionhip_ctx *ctx, const aionhip_weight *w, const unsigned short **out) {
    auto it = ctx->bf16_copies.find(w);
    if (it != ctx->bf16_copies.end()) {
        *out = (const unsigned short *)it->second.first;
        return AIONHIP_OK;
    }
    if (ctx->capturing)
        return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "the bf16 copy of a weight cannot be built while a program is being recorded: run the steps once before recording");
    const size_t N = w->n, K = w->k, rows_padded = (N + 15) & ~(size_t)15, bytes = rows_padded * K * 2;
    void *p = nullptr;
    int rc = dev_malloc(ctx, &p, bytes, "the bf16 copy of a weight");
    if (rc) return rc;
    const size_t threads = rows_padded * (K / 8);
    const unsigned grid = (unsigned)((threads + 255) / 256);
    if (w->dtype == AIONHIP_Q8_0) dequant_bf16_kernel<AIONHIP_Q8_0><<<dim3(grid), dim3(256), 0, ctx->stream>>>(w->qs, w->sc, (unsigned short *)p, N, K);
    else dequant_bf16_kernel<AIONHIP_Q4_0><<<dim3(grid), dim3(256), 0, ctx->stream>>>(w->qs, w->sc, (unsigned short *)p, N, K);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        (void)hipFree(p);
        return set_err(ctx, AIONHIP_EXECUTION_FAILED, "launch dequant_bf16: %s", hipGetErrorString(e));
    }
    ctx->bf16_copies[w] = {p, bytes};
    ctx->bf16_copy_bytes += bytes;
    *out = (const unsigned short *)p;
    return AIONHIP_OK;
}

int launch_gemm_bf16(aionhip_ctx *ctx, const aionhip_weight *w, size_t m, const float *a, size_t lda, float *c, size_t ldc, float alpha, float beta) {
    const size_t N = w->n, K = w->k;
    if ((((uintptr_t)a) & 3) != 0) return set_err(ctx, AIONHIP_INVALID_ARGUMENT, "gemm: A must be 4-byte aligned");
    // Two forms of the weight operand. With copies (the default) the kernel streams a bf16 copy of the weight that this
    // context builds on the weight's first bf16 call and keeps: 2 bytes per weight resident, and the faster kernel
    // (M = 2048 x N = 14336 x K = 4096, q4: 197 us). Without, the same kernel converts the quant blocks while it stages
    // them: nothing resident, nothing allocated, 264 us - the conversion's vector instructions, the LDS writes and the
    // scattered 16-byte requests all land in a loop that is already bound by instruction issue and power.
    const unsigned short *wcopy = nullptr;
    if (ctx->bf16_copies_on) {
        const int rc0 = bf16_copy_of(ctx, w, &wcopy);
        if (rc0) return rc0;
    }
    const size_t m_padded = (m + 15) & ~(size_t)15;
    int rc = ensure_scratch2(ctx, m_padded * K * 2);
    if (rc) return rc;
    unsigned short *abf = (unsigned short *)ctx->scratch2;
    {
        const size_t threads = m_padded * (K / 8);                 // = 64 lanes per (16 rows, 32 k) block
        ProfScope scope(ctx, "act_bf16");
        if ((((uintptr_t)a) & 15) == 0 && (lda & 3) == 0)
            launch_k(ctx, act_bf16_kernel<true>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, a, lda, abf, m, K);
        else
            launch_k(ctx, act_bf16_kernel<false>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, a, lda, abf, m, K);
        LAUNCH_CHECK(ctx, "act_bf16");
    }
    ProfScope scope(ctx, "gemm_bf16");
    {
        const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
        const int tn = (int)((N + G2_BN - 1) / G2_BN);
        // tallest tile that still gives every CU a workgroup; 64-row tiles when even 128-row ones leave half idle
        const int tm4 = (int)((m + 255) / 256), tm2 = (int)((m + 127) / 128), tm1 = (int)((m + 63) / 64);
        int wm = (long)tm4 * tn >= cus ? 4 : ((long)tm2 * tn * 2 > cus && (long)tm1 * tn > cus ? 2 : 1);   // (64-row tiles while they fit one round)
        // 256-row tiles come 256 or 192 columns wide (a 192-column tile takes 3/4 of the time). Three covers of N are weighed
        // by their rounds: whole rounds of wide tiles with the columns left over in one round of narrow ones; wide tiles only;
        // narrow tiles only (N = 11008 at 2048 rows: 58 narrow column tiles are two rounds of 3/4 where 32 wide + 15 narrow are
        // 1 + 3/4). Narrow tiles only also replace 128-row tiles that would need two half-time rounds where one round of
        // 256 x 192 tiles covers N (N = 5120 ... 6144 at 2048 rows).
        int tn_wide = tn, tn_narrow = 0;
        const int all_narrow = (int)((N + 191) / 192);
        if (wm == 2 && (long)tm4 * all_narrow <= cus && (long)tm2 * tn > cus) {
            wm = 4;
            tn_wide = 0;
            tn_narrow = all_narrow;
        } else if (wm == 4) {
            const int per_round = cus / tm4;                    // column tiles per round
            const int rest = per_round > 0 ? tn % per_round : 0;
            if (per_round > 0) {
                float best = (float)((tn + per_round - 1) / per_round);            // wide tiles only
                if (rest > 0 && tn > per_round) {
                    const size_t cols_left = N - (size_t)(tn - rest) * G2_BN;
                    const int narrow = (int)((cols_left + 191) / 192);
                    if ((long)narrow * tm4 <= cus && (float)((tn - rest) / per_round) + 0.75f <= best) {
                        best = (float)((tn - rest) / per_round) + 0.75f;
                        tn_wide = tn - rest;
                        tn_narrow = narrow;
                    }
                }
                const float narrow_only = 0.75f * (float)((all_narrow + per_round - 1) / per_round);
                if (narrow_only < best) {
                    best = narrow_only;
                    tn_wide = 0;
                    tn_narrow = all_narrow;
                }
                // barely more 256-row tiles than CUs: two half-time rounds of 128-row tiles beat a second round of tall ones
                // (1300 rows x 11008 columns: 258 tall tiles, 139 us; 473 of 128 rows, 115 us; a third, nearly empty half round
                // costs more than it saves: 516 tiles of 128 rows took 166 against 145 us)
                if (best > 1.f && (long)tm2 * tn <= 2L * cus) {
                    wm = 2;
                    tn_wide = tn;
                    tn_narrow = 0;
                }
            }
        }
        const int tm = wm == 4 ? tm4 : (wm == 2 ? tm2 : tm1);
        // 64-row tiles that still leave CUs idle (few tokens against a narrow weight): 128 columns instead of 256, twice the workgroups
        const bool half_cols = wm == 1 && (long)tm1 * tn < cus;
        // kernel variant: 0 = the bf16 copy, 1 = q4 blocks converted while staged, 2 = q8 blocks
        const int var = wcopy ? 0 : (w->dtype == AIONHIP_Q8_0 ? 2 : 1);
        const uint8_t *wp = wcopy ? (const uint8_t *)wcopy : w->qs;
        static bool attr[3][5] = {};
        auto launch = [&](auto kernel, int shape, int lds, int tiles) -> int {
            if (!attr[var][shape]) {
                HIP_TRY(ctx, hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
                attr[var][shape] = true;
            }
            launch_k(ctx, kernel, dim3((unsigned)((tiles + 7) / 8 * 8)), dim3(256), lds, abf, wp, w->sc, c, (int)m, (int)N, (int)K, ldc, alpha, beta, tm, tiles);
            return AIONHIP_OK;
        };
        auto launch_mixed = [&](auto kernel, int lds, int tiles) -> int {
            if (!attr[var][4]) {
                HIP_TRY(ctx, hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
                attr[var][4] = true;
            }
            launch_k(ctx, kernel, dim3((unsigned)((tiles + 7) / 8 * 8)), dim3(256), lds, abf, wp, w->sc, c, (int)m, (int)N, (int)K, ldc, alpha, beta,
                     tm, tn_wide, tn_narrow);
            return AIONHIP_OK;
        };
        auto with_variant = [&](auto f) -> int {
            if (var == 0) return f(std::integral_constant<int, 0>{});
            if (var == 1) return f(std::integral_constant<int, AIONHIP_Q4_0>{});
            return f(std::integral_constant<int, AIONHIP_Q8_0>{});
        };
        if (tn_narrow) {
            // both kinds of tiles in one launch, interleaved (gemm_bf16_mixed_kernel)
            rc = with_variant([&](auto b) { return launch_mixed(gemm_bf16_mixed_kernel<4, decltype(b)::value>, 4 * (256 + 256) * G2_ROW, tm * (tn_wide + tn_narrow)); });
        } else if (wm == 4) {
            rc = with_variant([&](auto b) { return launch(gemm_bf16_wide_kernel<4, 4, 4, decltype(b)::value>, 0, 4 * (256 + 256) * G2_ROW, tm * tn_wide); });
        } else if (wm == 2) {
            rc = with_variant([&](auto b) { return launch(gemm_bf16_wide_kernel<2, 4, 4, decltype(b)::value>, 1, 4 * (128 + 256) * G2_ROW, tm * tn_wide); });
        } else if (half_cols) {
            rc = with_variant([&](auto b) { return launch(gemm_bf16_wide_kernel<1, 4, 2, decltype(b)::value>, 3, 4 * (64 + 128) * G2_ROW, tm * (int)((N + 127) / 128)); });
        } else {
            rc = with_variant([&](auto b) { return launch(gemm_bf16_wide_kernel<1, 4, 4, decltype(b)::value>, 2, 4 * (64 + 256) * G2_ROW, tm * tn_wide); });
        }
        if (rc) return rc;
    }
    LAUNCH_CHECK(ctx, "gemm_bf16");
    return AIONHIP_OK;
}
