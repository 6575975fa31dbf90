// Pieces shared by the tiled W8A8 GEMM kernels (gemm_tile256.hip: INT8; gemm_tile_fp8.hip: FP8): fragment types, the
// tile a workgroup computes, the epilogue for accumulators held as 16x16 blocks, and the cut of a launch's last,
// partial round of workgroups.
#pragma once

#include "gemm_common.h"

namespace daxq {

template <bool FP8>
struct Frag {
    typedef v4i type;
};
template <>
struct Frag<true> {
    typedef v8i type;
};

struct Yes {
    static constexpr bool value = true;
};
struct No {
    static constexpr bool value = false;
};
template <int N>
struct Int {
    static constexpr int value = N;
};

// sched_group_barrier masks
#define DAXQ_SG_MFMA 0x008
#define DAXQ_SG_DS_RD 0x100

// GemmArgs::order
constexpr int kOrderRowGroups = 0, kOrderBanded = 1;

// Which BT x BT output tile workgroup `tile_id` computes: its origin (m0, n0), shifted inwards at the M / N edge
// instead of being predicated (the overlap rows are computed twice with identical results).  False: a padding slot of
// the banded order, the workgroup exits at once.  With quad_base > 0, BT = 128 means the four quadrants of the
// 256x256 tiles from id quad_base - 1 on, one workgroup per quadrant (tile_id counts quadrants).
template <int BT>
__device__ __forceinline__ bool tile_origin(const GemmArgs& p, int tile_id, int& m0, int& n0) {
    int tm, tn;
    if (BT == 128 && p.quad_base) {
        tile_of_block(p.gm, p.quad_base - 1 + (tile_id >> 2), p.tiles_m, p.tiles_n, tm, tn);  // the 256x256 tile
        m0 = tm * 256, n0 = tn * 256;
        m0 = (m0 + 256 <= p.m ? m0 : p.m - 256) + ((tile_id >> 1) & 1) * 128;
        n0 = (n0 + 256 <= p.n ? n0 : p.n - 256) + (tile_id & 1) * 128;
        return true;
    }
    if (p.order == kOrderBanded) {
        if (!tile_of_block_banded(tile_id, p.tiles_m, p.tiles_n, 4, tm, tn)) return false;
    } else {
        tile_of_block(p.gm, tile_id, p.tiles_m, p.tiles_n, tm, tn);
    }
    m0 = tm * BT, n0 = tn * BT;
    m0 = m0 + BT <= p.m ? m0 : p.m - BT;
    n0 = n0 + BT <= p.n ? n0 : p.n - BT;
    return true;
}

// workgroups of a launch of 256x256 tiles in the tile order a.order
static inline int64_t grid_of_order(const GemmArgs& a) {
    const int64_t tiles = (int64_t)a.tiles_m * a.tiles_n;
    if (a.order != kOrderBanded) return tiles;
    // the patch arithmetic of the banded order is 32-bit: beyond 2^30 tiles none of it runs and the caller's check of the
    // grid size refuses the launch
    return tiles <= (1 << 30) ? banded_grid(a.tiles_m, a.tiles_n, 4) : (int64_t)1 << 40;
}

// accumulators of one 16x16 block: int32 (v_mfma_i32_16x16x64_i8) or fp32 (v_mfma_f32_16x16x128_f8f6f4)
template <bool FP8>
struct Acc16 {
    typedef v4i type;
};
template <>
struct Acc16<true> {
    typedef v4f type;
};

// The epilogue of a wavefront's accumulators held as NBJ x NBI blocks of 16x16 (v_mfma_i32_16x16x64_i8,
// v_mfma_f32_16x16x128_f8f6f4): acc[j][i] is weight block j (16 output columns) and activation block i (16 output rows)
// of the wavefront's part of a tile of 32 NBI rows x 32 NBJ columns (four wavefronts, 2 x 2).
// In a block a lane owns output row m = l%16 and the columns n = 4*(l/16) + {0..3}.  One
// v_permlane16_swap per word over two neighbouring blocks gives each lane 8 consecutive columns of one
// of them: lanes 0-15 block 2jp columns 0-7, lanes 16-31 block 2jp+1 columns 0-7, lanes 32-47 block
// 2jp columns 8-15, lanes 48-63 block 2jp+1 columns 8-15.
// NBJ, NBI: 8, 8 for a 256x256 tile, 4, 4 for a 128x128 tile, 4, 8 for a half tile of 256 rows x 128 columns.
// OUTK: element type of out and bias, DAXQ_BF16 / DAXQ_F16 / DAXQ_F32.  A template argument, i.e. a kernel
// of its own per type: with all three forms inside one kernel behind uniform branches its code grew from 27 to 44 KB
// and the bf16 launches at K = 1536, which change between main loop and epilogue every 24 slices, lost 2.7 %; with
// the choice inside the loops they lost 2 to 11 % everywhere.
template <bool DUMP, int NBJ, int NBI, bool FP8 = false, int OUTK = DAXQ_BF16>
__device__ __forceinline__ void tile_epilogue16(const GemmArgs& p, typename Acc16<FP8>::type (&acc)[NBJ][NBI], uint8_t* smem, int m0, int n0, int t,
                                                int wm, int wn, int l15, int g4, float pre_sx, float pre_sw,
                                                float pre_bias) {
    constexpr int BM = 32 * NBI, BN = 32 * NBJ, WTM = 16 * NBI, WTN = 16 * NBJ;
    float* s_sx = reinterpret_cast<float*>(smem);
    float* s_sw = s_sx + BM;
    float* s_bias = s_sw + BN;
    if (BM == 256 || t < BM) s_sx[t] = pre_sx;
    if (BN == 256 || t < BN) {
        s_sw[t] = pre_sw;
        s_bias[t] = pre_bias;
    }
    __syncthreads();

    if constexpr (DUMP) {
#pragma unroll
        for (int j = 0; j < NBJ; ++j)
#pragma unroll
            for (int i = 0; i < NBI; ++i) {
                const int64_t m = m0 + wm * WTM + i * 16 + l15;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    if constexpr (FP8) static_cast<float*>(p.acc)[m * p.ldacc + n0 + wn * WTN + j * 16 + 4 * g4 + v] = acc[j][i][v];
                    else static_cast<int32_t*>(p.acc)[m * p.ldacc + n0 + wn * WTN + j * 16 + 4 * g4 + v] = acc[j][i][v];
                }
            }
    }

    float sxr[NBI];
    float4 swr[NBJ], br[NBJ];
#pragma unroll
    for (int i = 0; i < NBI; ++i) sxr[i] = s_sx[wm * WTM + i * 16 + l15];
#pragma unroll
    for (int j = 0; j < NBJ; ++j) {
        const int nl = wn * WTN + j * 16 + 4 * g4;
        swr[j] = *reinterpret_cast<const float4*>(s_sw + nl);
        br[j] = *reinterpret_cast<const float4*>(s_bias + nl);
    }
    __builtin_amdgcn_sched_barrier(0);

    // fp32 module: one rounding less and four-byte outputs, a lane's four columns of a block as one store
    if constexpr (OUTK == DAXQ_F32) {
        {
#pragma unroll
            for (int i = 0; i < NBI; ++i) {
                const float sxv = sxr[i];
                float* orow = reinterpret_cast<float*>(p.out) + (int64_t)(m0 + wm * WTM + i * 16 + l15) * p.ldo + n0 + wn * WTN + 4 * g4;
#pragma unroll
                for (int j = 0; j < NBJ; ++j) {
                    const float sws[4] = {swr[j].x, swr[j].y, swr[j].z, swr[j].w};
                    const float bs[4] = {br[j].x, br[j].y, br[j].z, br[j].w};
                    float o[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        float y = (float)acc[j][i][r];  // (int8: v_cvt_f32_i32, round to nearest even)
                        y = y * sxv;
                        y = y * sws[r];
                        o[r] = y + bs[r];
                    }
                    *reinterpret_cast<float4*>(orow + j * 16) = make_float4(o[0], o[1], o[2], o[3]);
                }
            }
        }
        return;
    }
    // out and bias are fp16 instead of bf16
    constexpr bool f16 = OUTK == DAXQ_F16;
    {
#pragma unroll
    for (int i = 0; i < NBI; ++i) {
        const int ml = wm * WTM + i * 16 + l15;
        const float sxv = sxr[i];
        uint16_t* orow = p.out + (int64_t)(m0 + ml) * p.ldo + n0 + wn * WTN + (g4 & 1) * 16 + (g4 >> 1) * 8;
#pragma unroll
        for (int jp = 0; jp < NBJ / 2; ++jp) {
            uint32_t pk[2][2];
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
                const int j = 2 * jp + jj;
                const float sws[4] = {swr[j].x, swr[j].y, swr[j].z, swr[j].w};
                const float bs[4] = {br[j].x, br[j].y, br[j].z, br[j].w};
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int r = 2 * h;
                    if constexpr (FP8) {
                        float z0 = acc[j][i][r] * sxv * sws[r] + bs[r], z1 = acc[j][i][r + 1] * sxv * sws[r + 1] + bs[r + 1];
                        if constexpr (f16) {  // one rounding, to fp16 (kept apart from the add: no mixed-precision fold)
                            asm("" : "+v"(z0), "+v"(z1));
                            pk[jj][h] = pack_f16_rne(z0, z1);
                        } else {
                            pk[jj][h] = pack_bf16_rne(z0, z1);
                        }
                    } else {
                        float y0 = (float)acc[j][i][r];  // v_cvt_f32_i32, round to nearest even
                        float y1 = (float)acc[j][i][r + 1];
                        y0 = y0 * sxv;
                        y1 = y1 * sxv;
                        y0 = y0 * sws[r];
                        y1 = y1 * sws[r + 1];
                        if constexpr (f16) {  // fp16 module: the same two roundings, to fp16
                            // (the products and sums pass through empty asm statements: the compiler otherwise folds
                            // a multiply or add and the conversion behind it into one mixed-precision instruction
                            // that rounds once, where the reference rounds to fp32 first)
                            asm("" : "+v"(y0), "+v"(y1));
                            float z0 = (float)(_Float16)y0 + bs[r], z1 = (float)(_Float16)y1 + bs[r + 1];
                            asm("" : "+v"(z0), "+v"(z1));
                            pk[jj][h] = pack_f16_rne(z0, z1);
                        } else {
                            const uint32_t o1 = pack_bf16_rne(y0, y1);
                            // second rounding: the bias is added to the bf16 value
                            pk[jj][h] = pack_bf16_rne(__uint_as_float(o1 << 16) + bs[r], __uint_as_float(o1 & 0xffff0000u) + bs[r + 1]);
                        }
                    }
                }
            }
            v2u s0 = __builtin_amdgcn_permlane16_swap(pk[0][0], pk[1][0], false, false);
            v2u s1 = __builtin_amdgcn_permlane16_swap(pk[0][1], pk[1][1], false, false);
            *reinterpret_cast<uint4*>(orow + jp * 32) = make_uint4(s0.x, s1.x, s0.y, s1.y);
        }
    }
    }
}

// CUs of the current device (0 if the query fails), asked once per device
static inline int cu_count() {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (dev >= 0 && dev < 64) {
        if (int c = cached[dev].load(std::memory_order_relaxed)) return c;
    }
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return 0;
    if (dev >= 0 && dev < 64) cached[dev].store(cus, std::memory_order_relaxed);
    return cus;
}

// Tiles of the last, partial round of a 256x256 launch that run as 128x128 quadrants, in workgroups behind those of
// the whole tiles; 0 = none.
// One workgroup of 256x256 tiles fills a CU, so a launch of R whole rounds and L more tiles takes R + 1 tile times
// however small L is.  As 4 L quadrants with a CU each (L <= a quarter of the CUs) the L tiles take half a tile time
// or less.  Measured as a second launch against the launch of whole tiles (INT8 / e4m3, K = 5120 unless noted; in one
// grid the quadrants start on the first CUs that come free, another +1 to +10 %, most on short launches):
//   4725 x 13824 (4 rounds + 2 tiles) +5.6 / +6.1 %; 8500 x 4096, K = 2048 (2 + 32) +9.9 / +9.9 %;
//   4095 x 4608, K = 1536 (1 + 32) +10.7 / +9.8 %, K = 8960 +24 / +26 %;
//   20000 x 5120 (6 + 44) +3.3 / +2.4 %; 75600 x 5120 in row groups (23 + 32) -0.6 / -0.8 %: over many rounds the CUs
//   drift apart and the early ones pick the last tiles up, so the cut is taken up to kTailMaxRounds whole rounds;
//   with two quadrants per CU (L up to half the CUs: 4725 x 5120, 1 + 124) -5.3 / -5.9 %: a round of 128x128 tiles
//   at two per CU takes as long as a round of 256x256 tiles, so those launches stay whole.
constexpr int kTailMaxRounds = 8;
static inline int tail_tiles(const GemmArgs& a, int tail) {
    if (tail == 1 || a.order != kOrderRowGroups) return 0;  // the banded order deals whole patches: its ids are not tile counts
    const int cus = cu_count();
    if (cus < 8) return 0;
    const int64_t tiles = (int64_t)a.tiles_m * a.tiles_n, rounds = tiles / cus, left = tiles - rounds * cus;
    if (rounds < 1 || left == 0 || 4 * left > cus) return 0;
    return (tail == 2 || rounds <= kTailMaxRounds) ? (int)left : 0;
}
// The same for a last round of more than a quarter and at most half of the CUs' worth of tiles: those run as halves of
// 256 x 128 with a CU each (gemm_tile256x128.h), about 0.65 of a tile time instead of one.
static inline int tail_half_tiles(const GemmArgs& a, int tail) {
    if (tail == 1 || a.order != kOrderRowGroups) return 0;
    const int cus = cu_count();
    if (cus < 8) return 0;
    const int64_t tiles = (int64_t)a.tiles_m * a.tiles_n, rounds = tiles / cus, left = tiles - rounds * cus;
    if (rounds < 1 || 4 * left <= cus || 2 * left > cus) return 0;
    return (tail == 2 || rounds <= kTailMaxRounds) ? (int)left : 0;
}

}  // namespace daxq
