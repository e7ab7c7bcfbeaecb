// 3..8 activation rows against q4_0 / q8_0 weights on the matrix pipe: gemv_mfma_kernel.
//
// The arithmetic is the one of every matmul here (aion cpu/kernels/matmul_q_i8.zig:436-470): per quant block an exact int32
// dot of int8 activation codes with the weight codes, then acc += f32(idot) * (a_scale * w_scale). With 4..8 activation rows the
// vector-ALU form (gemv_rows_kernel: eight dot4 per block per row pair) spends more issue slots on dots than the memory system
// needs to deliver the weights; here one v_mfma_i32_16x16x64_i8 does the dots of 16 weight rows for TWO quant blocks and up to
// 8 activation rows, and the vector ALU is left with the rescale: 3 operations per output, 4 outputs per lane per block pair.
//
//   A operand (16 x 64)  activation codes, block-diagonal: rows 0..7 hold the codes of block kb in k 0..31 and zeros in k 32..63,
//                        rows 8..15 zeros in k 0..31 and the codes of block kb+1 (the same 8 activation rows) in k 32..63.
//                        Lane (row l & 15, k group l >> 4) holds 16 consecutive codes - real ones or zeros.
//   B operand (64 x 16)  weight codes of 16 consecutive weight rows, blocks kb and kb+1 one after the other. q4: the lane's
//                        two dwords of a block's 16 bytes, low and high nibbles apart (the device layout pairs them with the
//                        activation codes in exactly that order); nibbles stay 0..15, -8 * sum(activation codes) enters as C.
//   D (16 x 16 int32)    rows 0..7: the exact block dots of block kb, rows 8..15: those of block kb+1 (K = 32 of each block
//                        meets zeros in the other block's rows). Lane (weight row l & 15, group g) holds activation rows
//                        4(g & 1) .. +3 of block kb + (g >> 1): every lane rescales and accumulates real results, and the two
//                        lane halves are added once per tile.
//
// Weights never pass through registers on their way in: every wavefront owns a ring of NSTG stages in LDS, a stage being 8
// quant blocks of its 16 rows plus their f16 scales, filled by LDS-writing loads (whole 128-byte lines per row) and waited
// for by count. The 16-byte chunks of a row are XOR-swizzled on the global side so that the operand reads of the 64 lanes
// fall into distinct banks. The activations (codes, scales, -8 * sums) of the launch's K range sit in LDS once per
// workgroup, shared by its four wavefronts and by every tile the workgroup walks (persistent grid).
// KS wavefronts share a tile when there are few weight rows, each taking every KS-th stage; their partial sums are added in
// wavefront order through LDS, so the result does not depend on timing.
#include "common.h"

namespace {

using i32x4 = __attribute__((ext_vector_type(4))) int;
using u32x2 = __attribute__((ext_vector_type(2))) unsigned int;

constexpr int MF_ROWS = 16, MF_SB = 8;          // weight rows per tile, quant blocks per stage
template <int DT>
struct MfCfg {
    static constexpr bool Q8 = DT == AIONHIP_Q8_0;
    static constexpr int ROWB = MF_SB * (Q8 ? 32 : 16);      // bytes of a row per stage
    static constexpr int CPR = ROWB / 16;                    // 16-byte chunks per row
    static constexpr int RPI = 64 / CPR;                     // rows one load instruction covers
    static constexpr int NLD = MF_ROWS / RPI;                // weight load instructions per stage
    static constexpr int W_BYTES = MF_ROWS * ROWB;
    static constexpr int STAGE = W_BYTES + MF_ROWS * MF_SB * 2;   // + the f16 scales: [16 rows][8 blocks]
    static constexpr int PER_BLOCK = 8 * 32 + 8 * 4 + (Q8 ? 0 : 8 * 4);   // LDS bytes of activations per quant block
};

struct MfSeg {
    const uint8_t *qs;
    const __half *sc;
    float *c;
    size_t ldc;
    int n, first_tile;
};
struct MfBatch {
    MfSeg seg[4];
    int count, tiles;
};

template <int DT, int NSTG, int KS>
__global__ __launch_bounds__(256) void gemv_mfma_kernel(MfBatch batch, const u32x4 *__restrict__ aq, const float *__restrict__ a_scale,
                                                        const int *__restrict__ a_sum, int K, int m, int kb0, int kbn, float alpha, float beta) {
    using Cfg = MfCfg<DT>;
    constexpr bool Q8 = Cfg::Q8;
    extern __shared__ __attribute__((aligned(1024))) unsigned char s_mf[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, g = lane >> 4;
    const int KB = K >> 5;
    // LDS: [wave rings][activation codes: kbn x 8 rows x 32 B][scales: kbn x 8 f32][q4: -8 * sums: kbn x 8 i32][KS > 1: partial sums][16 zero bytes]
    unsigned char *ring = s_mf + wave * (NSTG * Cfg::STAGE);
    unsigned char *s_act = s_mf + 4 * NSTG * Cfg::STAGE;
    float *s_as = (float *)(s_act + (size_t)kbn * 256);
    int *s_bias = (int *)(s_as + kbn * 8);

    constexpr int TPW = 4 / KS;                                  // tiles a workgroup works on at once
    const int kpart = wave % KS;
    const int stages = kbn / MF_SB;                              // the launcher passes whole stages only
    const int my_stages = (stages - kpart + KS - 1) / KS;        // stages kpart, kpart + KS, ...
    const size_t row_bytes = Q8 ? (size_t)K : (size_t)(K >> 1);

    // per-lane constants of the loads: instruction j of a stage covers rows j*RPI .. +RPI; lane -> (row, slot);
    // the slot holds chunk slot ^ swz(row) of the row's bytes of this stage
    const int l_row = lane / Cfg::CPR, l_slot = lane % Cfg::CPR;
    auto swz = [](int row) { return Q8 ? (row & 15) : ((row >> 1) & 7); };

    struct Tile {
        const uint8_t *wrow[Cfg::NLD];      // this lane's row of each load instruction, at the launch's first block
        const unsigned char *srow;          // this lane's piece of the scales: row lane >> 2, blocks 2 * (lane & 3) ..
        int seg, row0, valid;
    };
    auto open_tile = [&](int tile) {
        Tile t;
        t.valid = tile < batch.tiles;
        const int tc = t.valid ? tile : batch.tiles - 1;
        int si = 0;
#pragma unroll
        for (int i = 1; i < 4; ++i)
            if (i < batch.count && tc >= batch.seg[i].first_tile) si = i;
        t.seg = si;
        const int N = batch.seg[si].n;
        t.row0 = (tc - batch.seg[si].first_tile) * MF_ROWS;
#pragma unroll
        for (int j = 0; j < Cfg::NLD; ++j) {
            const int rl = j * Cfg::RPI + l_row;
            const int row = min(t.row0 + rl, N - 1);
            t.wrow[j] = batch.seg[si].qs + (size_t)row * row_bytes + (size_t)kb0 * (Q8 ? 32 : 16) + ((l_slot ^ swz(rl)) * 16);
        }
        t.srow = (const unsigned char *)(batch.seg[si].sc + (size_t)min(t.row0 + (lane >> 2), N - 1) * KB + kb0) + (lane & 3) * 4;
        return t;
    };
    auto issue_stage = [&](const Tile &t, int k, int slot) {       // k: k-th stage of this wavefront (clamped: a repeat lands in a dead slot)
#if defined(__HIP_DEVICE_COMPILE__)
        const int st = min(kpart + k * KS, stages - 1);
        unsigned char *dst = ring + slot * Cfg::STAGE;
#pragma unroll
        for (int j = 0; j < Cfg::NLD; ++j)
            __builtin_amdgcn_global_load_lds(t.wrow[j] + (size_t)st * Cfg::ROWB, (lds_void *)(dst + j * 1024), 16, 0, 0);
        __builtin_amdgcn_global_load_lds(t.srow + st * (MF_SB * 2), (lds_void *)(dst + Cfg::W_BYTES), 4, 0, 0);
#endif
    };
    constexpr int LPS = Cfg::NLD + 1;                             // load instructions per stage

    const int wg_first = blockIdx.x * TPW, tile_stride = gridDim.x * TPW;
    Tile cur = open_tile(wg_first + wave / KS);

    // ---- activations of the K range -> LDS, rows m..7 zero. The first batch of their loads is requested, then the first
    // stages of the first tile (both in flight together; the loads retire in order, so the activation data is waited for
    // by count without draining the ring), then the copy goes on.
    // Ring slots are used round robin across tiles: rs is the slot of the next stage to consume.
    int rs = 0;
    {
        const int chunks = kbn * 2;                               // 16-byte chunks per activation row
        const int a_chunks = K >> 4;
        const int total = 8 * chunks;
        constexpr int AB = 8, SBT = 2;                            // loads per thread in flight: 8 rows x 4096 codes in one batch
        const int quads = kbn >> 2, total_q = 8 * quads;          // scales and sums: four consecutive blocks of a row per load
        for (int base = 0, base_q = 0; base < total || base_q < total_q; base += 256 * AB, base_q += 256 * SBT) {
            u32x4 v[AB];
            f32x4 sv[SBT];
            i32x4 bv[SBT];
            if (base < total) {
#pragma unroll
                for (int i = 0; i < AB; ++i) {
                    const int idx = min(base + tid + 256 * i, total - 1);
                    const int b = idx / chunks, c = idx - b * chunks;
                    v[i] = aq[(size_t)min(b, m - 1) * a_chunks + 2 * kb0 + c];   // unconditional: a load under a branch is waited for on the spot
                }
            }
            if (base_q < total_q) {
#pragma unroll
                for (int i = 0; i < SBT; ++i) {
                    const int idx = min(base_q + tid + 256 * i, total_q - 1);
                    const int b = idx / quads, qd = idx - b * quads;
                    sv[i] = *(const f32x4 *)(a_scale + (size_t)min(b, m - 1) * KB + kb0 + qd * 4);
                    if (!Q8) bv[i] = *(const i32x4 *)(a_sum + (size_t)min(b, m - 1) * KB + kb0 + qd * 4);
                }
            }
            if (base == 0) {
#pragma unroll
                for (int k = 0; k < NSTG - 1; ++k) issue_stage(cur, k, k);
            }
            if (base < total) {
#pragma unroll
                for (int i = 0; i < AB; ++i) {
                    const int idx = base + tid + 256 * i;
                    if (idx < total) {
                        const int b = idx / chunks, c = idx - b * chunks;
                        *(u32x4 *)(s_act + ((size_t)(c >> 1) * 8 + b) * 32 + (c & 1) * 16) = b < m ? v[i] : u32x4{0u, 0u, 0u, 0u};
                    }
                }
            }
            if (base_q < total_q) {
#pragma unroll
                for (int i = 0; i < SBT; ++i) {
                    const int idx = base_q + tid + 256 * i;
                    if (idx < total_q) {
                        const int b = idx / quads, qd = idx - b * quads;
                        const float se[4] = {sv[i].x, sv[i].y, sv[i].z, sv[i].w};
                        const int be[4] = {Q8 ? 0 : bv[i].x, Q8 ? 0 : bv[i].y, Q8 ? 0 : bv[i].z, Q8 ? 0 : bv[i].w};
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            s_as[(qd * 4 + e) * 8 + b] = b < m ? se[e] : 0.f;
                            if (!Q8) s_bias[(qd * 4 + e) * 8 + b] = b < m ? -8 * be[e] : 0;
                        }
                    }
                }
            }
        }
    }
    __syncthreads();

    const int hb = g >> 1, hh = g & 1;                             // which block of a pair this lane's k group and results belong to; which half of it
    const bool a_real = (n >> 3) == hb;                          // block-diagonal A: real codes, or zeros
    unsigned char *s_zero = (unsigned char *)(s_bias + (Q8 ? 0 : kbn * 8)) + (KS > 1 ? 4096 : 0);      // 16 zero bytes behind everything else
    if (tid < 4) ((unsigned *)s_zero)[tid] = 0u;
    const unsigned char *a_base = a_real ? s_act + (hb * 8 + (n & 7)) * 32 + hh * 16 : s_zero;
    const int a_step = a_real ? 512 : 0;                         // bytes per block pair
    const int s_off = hb * 8 + hh * 4;                           // this lane's four activation rows of its block, in floats from the pair's first
    const int w_off = Q8 ? n * Cfg::ROWB : n * Cfg::ROWB + hh * 8;
    const int w_swz = swz(n);
    const int ws_shift = hb * 16;
    float *red = (float *)(s_bias + (Q8 ? 0 : kbn * 8));           // KS > 1: [wave][lane] partial sums
    __syncthreads();                                             // the zero bytes

    for (int it = 0; wg_first + it * tile_stride < batch.tiles; ++it) {      // the same trip count for every wavefront of a workgroup
        const Tile next = open_tile(wg_first + wave / KS + (it + 1) * tile_stride);
        f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int k = 0; k < my_stages; ++k) {
            // keep NSTG - 1 stages in flight: past this tile's last stage, the next tile's first ones
            const int ahead = k + NSTG - 1;
            const int ws_slot = rs == 0 ? NSTG - 1 : rs - 1;       // the slot consumed last
            if (ahead < my_stages) issue_stage(cur, ahead, ws_slot);
            else issue_stage(next, ahead - my_stages, ws_slot);
            __builtin_amdgcn_s_waitcnt(vmcnt_imm((NSTG - 1) * LPS));
            const unsigned char *st = ring + rs * Cfg::STAGE;
            rs = rs + 1 == NSTG ? 0 : rs + 1;
            const int kb = (kpart + k * KS) * MF_SB;
            const u32x4 sc8 = *(const u32x4 *)(st + Cfg::W_BYTES + n * 16);
            const unsigned scw[4] = {sc8.x, sc8.y, sc8.z, sc8.w};
            // All of a stage's operands are requested, then its four MFMAs issued, then the rescales: one LDS round trip and
            // one MFMA latency per stage instead of one per block pair (the compiler, left alone, waits pair by pair).
            constexpr int NP = MF_SB / 2;
            u32x2 wv[NP];
            i32x4 wl[NP], av[NP], d[NP];
            f32x4 as4[NP];
            const unsigned char *ap = a_base + (size_t)a_step * (kb >> 1);
#pragma unroll
            for (int jj = 0; jj < NP; ++jj) {
                if (Q8) wl[jj] = *(const i32x4 *)(st + w_off + (((jj * 4 + g) ^ w_swz) * 16));
                else wv[jj] = *(const u32x2 *)(st + w_off + (((jj * 2 + hb) ^ w_swz) * 16));
                av[jj] = *(const i32x4 *)(ap + jj * a_step);
            }
#pragma unroll
            for (int jj = 0; jj < NP; ++jj) {
                d[jj] = i32x4{0, 0, 0, 0};
                if (!Q8) d[jj] = *(const i32x4 *)(s_bias + (kb + 2 * jj) * 8 + s_off);
                as4[jj] = *(const f32x4 *)(s_as + (kb + 2 * jj) * 8 + s_off);
            }
#pragma unroll
            for (int jj = 0; jj < NP; ++jj) {
                i32x4 b;
                if (Q8) b = wl[jj];
                else b = i32x4{(int)(wv[jj].x & 0x0F0F0F0Fu), (int)((wv[jj].x >> 4) & 0x0F0F0F0Fu), (int)(wv[jj].y & 0x0F0F0F0Fu), (int)((wv[jj].y >> 4) & 0x0F0F0F0Fu)};
                d[jj] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av[jj], b, d[jj], 0, 0, 0);
            }
#pragma unroll
            for (int jj = 0; jj < NP; ++jj) {
                const float ws = __half2float(__ushort_as_half((unsigned short)(scw[jj] >> ws_shift)));
                acc.x += (float)d[jj].x * (as4[jj].x * ws);
                acc.y += (float)d[jj].y * (as4[jj].y * ws);
                acc.z += (float)d[jj].z * (as4[jj].z * ws);
                acc.w += (float)d[jj].w * (as4[jj].w * ws);
            }
        }
        // even blocks were accumulated by lanes 0..31, odd blocks by lanes 32..63: one add per tile
        acc.x += __shfl_xor(acc.x, 32, 64);
        acc.y += __shfl_xor(acc.y, 32, 64);
        acc.z += __shfl_xor(acc.z, 32, 64);
        acc.w += __shfl_xor(acc.w, 32, 64);
        // ---- the tile's results: lanes 0..31 (weight row n, group g) hold activation rows 4g .. 4g+3
        if (KS > 1) {
            *(f32x4 *)(red + (wave * 64 + lane) * 4) = acc;
            __syncthreads();
            if (kpart == 0) {
#pragma unroll
                for (int w = 1; w < KS; ++w) acc += *(const f32x4 *)(red + ((wave + w) * 64 + lane) * 4);
            }
            __syncthreads();                                     // the partial sums are read before the next tile writes its own
        }
        if (cur.valid && kpart == 0 && g < 2) {
            const MfSeg &sg = batch.seg[cur.seg];
            const int row = cur.row0 + n;
            if (row < sg.n) {
                const float v[4] = {acc.x, acc.y, acc.z, acc.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int b = g * 4 + i;
                    if (b < m) {
                        float *dst = sg.c + (size_t)b * sg.ldc + row;
                        const float o = alpha * v[i];
                        *dst = beta == 0.f ? o : o + beta * *dst;
                    }
                }
            }
        }
        cur = next;
    }
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));                    // no LDS-writing load may outlive the workgroup
}

template <int DT, int NSTG, int KS>
int launch_mf(aionhip_ctx *ctx, const MfBatch &batch, int wgs, size_t lds, const u32x4 *aq, PreparedAct act, int K, int m, int kb0, int kbn,
              float alpha, float beta) {
    static size_t attr = 0;                                       // per instantiation: the largest LDS size asked for so far
    if (lds > 64 * 1024 && lds > attr) {
        HIP_TRY(ctx, hipFuncSetAttribute((const void *)gemv_mfma_kernel<DT, NSTG, KS>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(160 * 1024)));
        attr = 160 * 1024;
    }
    launch_k(ctx, gemv_mfma_kernel<DT, NSTG, KS>, dim3((unsigned)wgs), dim3(256), lds, batch, aq, act.scale, act.sum, K, m, kb0, kbn, alpha, beta);
    return AIONHIP_OK;
}

template <int DT>
int launch_mf_dt(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, int m, PreparedAct act,
                 float alpha, float beta) {
    using Cfg = MfCfg<DT>;
    const int K = (int)ws[0]->k, KB = K >> 5, stages_all = KB / MF_SB;
    const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
    MfBatch batch{};
    batch.count = count;
    int tiles = 0;
    for (int i = 0; i < count; ++i) {
        batch.seg[i] = MfSeg{ws[i]->qs, ws[i]->sc, cs[i], ldcs[i], (int)ws[i]->n, tiles};
        tiles += ((int)ws[i]->n + MF_ROWS - 1) / MF_ROWS;
    }
    batch.tiles = tiles;
    // wavefronts per tile: one while that gives every CU four tiles, else the K range is shared by two
    int ks = tiles >= cus * 4 ? 1 : 2;
    while (ks > 1 && stages_all / ks < 8) ks >>= 1;               // too short a K to share
    const int wgs_all = (tiles * ks + 3) / 4;
    // Ring depth: 4 stages when two workgroups share a CU, 8 (q8: 4, a stage is twice the bytes) when a workgroup has the
    // CU to itself - about 48..56 KB of weight loads in flight per CU either way.
    const size_t red = (ks > 1 ? 4096 : 0) + 16;                  // partial sums of sibling wavefronts; the zero bytes of the A operand
    const size_t ring4 = 4 * 4 * (size_t)Cfg::STAGE, ring8 = 4 * 8 * (size_t)Cfg::STAGE;
    const size_t act_all = (size_t)KB * Cfg::PER_BLOCK;
    const bool two_per_cu = wgs_all > cus && ring4 + act_all + red <= 80 * 1024;
    const int nstg = two_per_cu || Cfg::Q8 ? 4 : 8;
    const size_t ring = nstg == 4 ? ring4 : ring8;
    // K ranges whose activations fit the LDS left over, as even as possible, whole stages each
    const size_t budget = (two_per_cu ? 80 : 158) * 1024 - ring - red;
    const int max_stages = (int)(budget / ((size_t)Cfg::PER_BLOCK * MF_SB));
    if (max_stages < stages_all) return -1;                      // the activations of the whole K do not fit the LDS left over
    if (stages_all / ks < nstg - 1) return -1;                   // shorter than the ring: the caller falls back
    const int wgs = (int)min((long)wgs_all, (long)cus * (two_per_cu ? 2 : 1));
    const auto *aq = (const u32x4 *)act.q;
    const int kbn = stages_all * MF_SB;
    const size_t lds = ring + (size_t)kbn * Cfg::PER_BLOCK + red;
    if (nstg == 4) return ks == 1 ? launch_mf<DT, 4, 1>(ctx, batch, wgs, lds, aq, act, K, m, 0, kbn, alpha, beta)
                                  : launch_mf<DT, 4, 2>(ctx, batch, wgs, lds, aq, act, K, m, 0, kbn, alpha, beta);
    return ks == 1 ? launch_mf<DT, 8, 1>(ctx, batch, wgs, lds, aq, act, K, m, 0, kbn, alpha, beta)
                   : launch_mf<DT, 8, 2>(ctx, batch, wgs, lds, aq, act, K, m, 0, kbn, alpha, beta);
}

}  // namespace

// Where this kernel is ahead of the vector-ALU rows kernel (and of the exact GEMM's 16-row tile), from a sweep of 3..8 rows over
// N = 14336 ... 262144 x K = 2048 ... 8192, both weight types: it needs many row tiles to amortise its longer start (ring fill
// behind the activation copy), and it gains most where the vector ALU is the rows kernel's bound - q4 from five rows on.
//   q4, 5..8 rows, N >= 14336: 14336 x 4096 19.3 against 20.1 us, 24576 x 4096 20.8 / 25.0, 65536 x 4096 33.0 / 41.9,
//                               262144 x 2048 60.0 / 83.6 (8 rows)
//   q4, 3..4 rows, N >= 65536: 65536 x 2048 20.5 / 23.5, 131072 x 2048 31.1 / 39.0, 262144 x 2048 62.2 / 66.6 (4 rows);
//                               below that the rows kernel leads (32768 x 4096: 22.3 / 21.1)
//   q8, 3..8 rows, N >= 65536 and up to 300 M weights: 65536 x 2048 28.5 / 31.1, 131072 x 2048 49.0 / 53.5, 65536 x 4096
//                               52.0 / 59.5; past that size the rows kernel streams faster (262144 x 2048: 107 / 99)
// K: whole 256-code stages, 2048 ... 4096 (at 8192 the rows kernel is far ahead at 3..4 rows, the exact GEMM even at 5..8).
// N counts the rows of all weights of the call (siblings share the launch).
bool gemv_mfma_applies(const aionhip_weight *const *ws, int count, int m) {
    if (m < 3 || m > 8 || count < 1 || count > 4) return false;
    const size_t k = ws[0]->k;
    if (k % (MF_SB * 32) != 0 || k < 2048 || k > 4096) return false;
    size_t rows = 0;
    for (int i = 0; i < count; ++i) {
        if (ws[i]->k != k || ws[i]->dtype != ws[0]->dtype || ws[i]->n < 1) return false;
        rows += ws[i]->n;
    }
    if (ws[0]->dtype == AIONHIP_Q4_0) return rows >= (m >= 5 ? (size_t)14336 : (size_t)65536);
    if (ws[0]->dtype == AIONHIP_Q8_0) return rows >= 65536 && rows * k <= (size_t)300 * 1000 * 1000;
    return false;
}

// returns -1 when the shape does not suit the kernel after all (the caller then takes the vector-ALU kernel)
int launch_gemv_mfma(aionhip_ctx *ctx, const aionhip_weight *const *ws, float *const *cs, const size_t *ldcs, int count, int m, PreparedAct act,
                     float alpha, float beta) {
    return ws[0]->dtype == AIONHIP_Q8_0 ? launch_mf_dt<AIONHIP_Q8_0>(ctx, ws, cs, ldcs, count, m, act, alpha, beta)
                                        : launch_mf_dt<AIONHIP_Q4_0>(ctx, ws, cs, ldcs, count, m, act, alpha, beta);
}
