// 256x256-tile W8A8 GEMMs for gfx950: the kernels the large DiT shapes run on.
//
// Three kernels on the same tile live here.  The library launches gemm_tile256s5_kernel for INT8 (K in 64-byte slices
// through five 32 KB LDS stages, v_mfma_i32_16x16x64_i8) and gemm_tile256f16_kernel for FP8 (K in pairs of such slices,
// v_mfma_f32_16x16x128_f8f6f4, B fragments refilled in place; at the end of the file).  gemm_tile256s5_kernel with
// 32x32 MFMAs (INT8 32x32x32, FP8 32x32x64) and gemm_tile256_kernel (K in 128-byte slices, two 64 KB stages; it came
// first) stay as further implementations for the tests and for K < 512 in FP8.
//
// Work decomposition
//   workgroup  256 x 256 outputs, 4 wavefronts (one per SIMD) in a 2 x 2 grid
//   wavefront  128 x 128 outputs in 256 accumulator registers (AGPRs): 4 x 4 MFMA blocks of 32x32
//              (the older forms) or 8 x 8 blocks of 16x16 (the kernels the library launches)
// A 2 x 2 wave grid is what minimises LDS reads per MFMA for a square tile: 128 bytes of K are
// read (2 + 2) * 256 * 128 B = 128 KB per workgroup against 4096 MFMA cycles per wave.
//
// Data movement of the two-stage form
//   HBM/L2 -> LDS   global_load_lds_dwordx4 (no VGPR staging): 16 per thread and slice.  The 16-byte
//                   chunk c of tile row r lands in LDS at chunk slot c ^ f(r); the swizzle is applied
//                   to the global address because the LDS side of a DMA load is fixed (64 lanes in a row)
//   LDS -> VGPR     ds_read_b128, bank-conflict free thanks to the swizzle, read one (FP8) or two
//                   (INT8) MFMA steps ahead into further fragment register sets
//   one s_barrier per K slice; the MFMA step after it is cut into 16 scheduling regions of one
//   MFMA + one DMA load + one fragment read so that the loads of slice kt+2 and the first
//   fragments of slice kt+1 are spread over its MFMAs.
//
// Which tile a workgroup computes is a launch argument (GemmArgs::order): groups of tile rows per XCD (tile_of_block,
// gemm_common.h) or one of the orders of tile_order.h that give the 32 CUs of an XCD a patch of 32 tiles; the large
// launches take the banded one (the eight XCDs on the same activation rows and on different weight columns).
//
// Tiles at the M / N edge are shifted inwards (origin min(tile*256, dim-256)) instead of being
// predicated: the overlap rows are computed twice with identical results.  The five-stage kernel
// also exists on 128x128 tiles (launches with too few 256-tiles to fill the CUs); shapes with
// M < 128 or N < 128 take the generic kernel in gemm_w8a8.hip.
#include "gemm_common.h"

namespace daxq {

namespace t256 {
constexpr int BM = 256, BN = 256, BK = 128, T = 256;
constexpr int A_BYTES = BM * BK, STAGE = (BM + BN) * BK;
constexpr int LOADS = (BM + BN) * BK / 16 / T;  // 16 per thread per slice
constexpr int SMEM = 2 * STAGE;
}  // namespace t256

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

// per-lane constants of the LDS -> MFMA operand reads
struct FragAddr {
    const uint8_t* a_rd;  // row (wm*128 + l%32) of the A part of buffer 0
    const uint8_t* b_rd;  // row (wn*128 + l%32) of the B part of buffer 0
    int hi, fl;           // K half l/32, swizzle f(l%32)
};

template <bool FP8>
__device__ __forceinline__ void load_frags(const FragAddr& fa, int stage, int ks, typename Frag<FP8>::type (&af)[4],
                                           typename Frag<FP8>::type (&bf)[4]) {
    using namespace t256;
    const uint8_t* pa = fa.a_rd + stage * STAGE;
    const uint8_t* pb = fa.b_rd + stage * STAGE;
    if constexpr (!FP8) {
        const int xo = ((ks * 2 + fa.hi) ^ fa.fl) << 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) af[i] = *reinterpret_cast<const v4i*>(pa + i * 32 * BK + xo);
#pragma unroll
        for (int j = 0; j < 4; ++j) bf[j] = *reinterpret_cast<const v4i*>(pb + j * 32 * BK + xo);
    } else {
        const int xo0 = ((ks * 4 + fa.hi * 2) ^ fa.fl) << 4, xo1 = ((ks * 4 + fa.hi * 2 + 1) ^ fa.fl) << 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v4i lo = *reinterpret_cast<const v4i*>(pa + i * 32 * BK + xo0);
            v4i up = *reinterpret_cast<const v4i*>(pa + i * 32 * BK + xo1);
            af[i] = __builtin_shufflevector(lo, up, 0, 1, 2, 3, 4, 5, 6, 7);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v4i lo = *reinterpret_cast<const v4i*>(pb + j * 32 * BK + xo0);
            v4i up = *reinterpret_cast<const v4i*>(pb + j * 32 * BK + xo1);
            bf[j] = __builtin_shufflevector(lo, up, 0, 1, 2, 3, 4, 5, 6, 7);
        }
    }
}

// one fragment of the next slice's step 0: g = 0..3 -> A block g, g = 4..7 -> B block g-4 (INT8: one
// ds_read_b128; FP8: two)
template <bool FP8>
__device__ __forceinline__ void load_one_frag(const FragAddr& fa, int stage, int g, typename Frag<FP8>::type (&af)[4],
                                              typename Frag<FP8>::type (&bf)[4]) {
    using namespace t256;
    const uint8_t* pr = (g < 4 ? fa.a_rd : fa.b_rd) + stage * STAGE + (g & 3) * 32 * BK;
    if constexpr (!FP8) {
        const int xo = (fa.hi ^ fa.fl) << 4;
        (g < 4 ? af[g & 3] : bf[g & 3]) = *reinterpret_cast<const v4i*>(pr + xo);
    } else {
        const int xo0 = ((fa.hi * 2) ^ fa.fl) << 4, xo1 = ((fa.hi * 2 + 1) ^ fa.fl) << 4;
        v4i lo = *reinterpret_cast<const v4i*>(pr + xo0);
        v4i up = *reinterpret_cast<const v4i*>(pr + xo1);
        (g < 4 ? af[g & 3] : bf[g & 3]) = __builtin_shufflevector(lo, up, 0, 1, 2, 3, 4, 5, 6, 7);
    }
}

// ZERO: the block's first MFMA of a tile, which starts from zero instead of the accumulator
// F8: FP8 operand formats (kF8XE5 / kF8WE5: e5m2 activation / weight bytes)
template <bool FP8, int F8, bool ZERO = false, int NB = 4>
__device__ __forceinline__ void mfma_one(typename AccT<FP8>::type (&acc)[NB][NB], int g, const typename Frag<FP8>::type (&af)[4],
                                         const typename Frag<FP8>::type (&bf)[4]) {
    const int j = g / NB, i = g % NB;
    typename AccT<FP8>::type c = {};
    if constexpr (!ZERO) c = acc[j][i];
    if constexpr (!FP8)
        acc[j][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[j], af[i], c, 0, 0, 0);
    else
        acc[j][i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf[j], af[i], c, (F8 & kF8WE5) ? 1 : 0, (F8 & kF8XE5) ? 1 : 0, 0, 0, 0, 0);
}

// acc[j][i]: 32x32 block with rows = n (W rows, MFMA "A" operand) and columns = m (X rows, "B"
// operand), so that a lane ends up owning one output row m and runs of 4 consecutive n.
// F8: e5m2 instead of e4m3fn bytes (format selects: weights are the MFMA "A" operand, activations the "B" operand).
template <bool FP8, int F8>
__device__ __forceinline__ void mfma_step(typename AccT<FP8>::type (&acc)[4][4], const typename Frag<FP8>::type (&af)[4],
                                          const typename Frag<FP8>::type (&bf)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if constexpr (!FP8)
                acc[j][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[j], af[i], acc[j][i], 0, 0, 0);
            else
                acc[j][i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf[j], af[i], acc[j][i], (F8 & kF8WE5) ? 1 : 0, (F8 & kF8XE5) ? 1 : 0, 0, 0, 0, 0);
        }
}

// Epilogue.  In a 32x32 block a lane owns output row m = l%32 and, in registers 4q..4q+3, the
// columns n = 8q + 4*(l/32) + {0..3}.  Two v_permlane32_swap per pair of q give each lane 8
// consecutive columns, stored as one 16-byte write.  The tile's scales and bias are staged in LDS.
// pre_*: this thread's element (index t) of the tile's sx / sw / bias, already loaded by the caller.
// NB: 32x32 blocks per operand and wavefront (4: 256x256 tile, 2: 128x128 tile); the tile edge is 64 * NB.
template <bool FP8, bool DUMP, int NB = 4>
__device__ __forceinline__ void tile256_epilogue(const GemmArgs& p, typename AccT<FP8>::type (&acc)[NB][NB], uint8_t* smem,
                                                 int m0, int n0, int t, int wm, int wn, int l31, int hi, float pre_sx,
                                                 float pre_sw, float pre_bias) {
    constexpr int BT = 64 * NB, WT = 32 * NB;
    float* s_sx = reinterpret_cast<float*>(smem);
    float* s_sw = s_sx + BT;
    float* s_bias = s_sw + BT;
    if (BT == 256 || t < BT) {
        s_sx[t] = pre_sx;
        s_sw[t] = pre_sw;
        s_bias[t] = pre_bias;
    }
    __syncthreads();

    if constexpr (DUMP) {
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                const int64_t m = m0 + wm * WT + i * 32 + l31;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int n = n0 + wn * WT + j * 32 + 8 * (v >> 2) + 4 * hi + (v & 3);
                    if constexpr (!FP8)
                        static_cast<int32_t*>(p.acc)[m * p.ldacc + n] = acc[j][i][v];
                    else
                        static_cast<float*>(p.acc)[m * p.ldacc + n] = acc[j][i][v];
                }
            }
    }

    // every scale and bias value this lane needs goes into registers in one burst of LDS reads
    // (the fragment registers of the main loop are free now): 4 x sx, 16 x 4 sw, 16 x 4 bias
    float sxr[NB];
    float4 swr[NB][4], br[NB][4];
#pragma unroll
    for (int i = 0; i < NB; ++i) sxr[i] = s_sx[wm * WT + i * 32 + l31];
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int nl = wn * WT + j * 32 + 8 * q + 4 * hi;
            swr[j][q] = *reinterpret_cast<const float4*>(s_sw + nl);
            br[j][q] = *reinterpret_cast<const float4*>(s_bias + nl);
        }
    __builtin_amdgcn_sched_barrier(0);

#pragma unroll
    for (int i = 0; i < NB; ++i) {
        const int ml = wm * WT + i * 32 + l31;
        const float sxv = sxr[i];
        uint16_t* orow = p.out + (int64_t)(m0 + ml) * p.ldo + n0 + wn * WT + 8 * hi;
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            uint32_t pk[4][2];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float sws[4] = {swr[j][q].x, swr[j][q].y, swr[j][q].z, swr[j][q].w};
                const float bs[4] = {br[j][q].x, br[j][q].y, br[j][q].z, br[j][q].w};
#pragma unroll
                for (int h = 0; h < 2; ++h) {  // two columns at a time: v_cvt_pk_bf16_f32 rounds a pair (RNE)
                    const int r = 2 * h;
                    if constexpr (!FP8) {
                        float y0 = (float)acc[j][i][q * 4 + r];  // v_cvt_f32_i32, round to nearest even
                        float y1 = (float)acc[j][i][q * 4 + r + 1];
                        y0 = y0 * sxv;
                        y1 = y1 * sxv;
                        y0 = y0 * sws[r];
                        y1 = y1 * sws[r + 1];
                        const uint32_t o1 = pack_bf16_rne(y0, y1);
                        // second rounding: the bias is added to the bf16 value
                        pk[q][h] = pack_bf16_rne(__uint_as_float(o1 << 16) + bs[r],
                                                 __uint_as_float(o1 & 0xffff0000u) + bs[r + 1]);
                    } else {
                        pk[q][h] = pack_bf16_rne(acc[j][i][q * 4 + r] * sxv * sws[r] + bs[r],
                                                 acc[j][i][q * 4 + r + 1] * sxv * sws[r + 1] + bs[r + 1]);
                    }
                }
            }
#pragma unroll
            for (int qp = 0; qp < 2; ++qp) {
                // lanes 0-31 keep their half of q=2qp and receive the upper lanes' half of it;
                // lanes 32-63 receive the lower lanes' half of q=2qp+1 and keep their own
                v2u s0 = __builtin_amdgcn_permlane32_swap(pk[2 * qp][0], pk[2 * qp + 1][0], false, false);
                v2u s1 = __builtin_amdgcn_permlane32_swap(pk[2 * qp][1], pk[2 * qp + 1][1], false, false);
                *reinterpret_cast<uint4*>(orow + j * 32 + 16 * qp) = make_uint4(s0.x, s1.x, s0.y, s1.y);
            }
        }
    }
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

// The same epilogue for accumulators held as 8 x 8 blocks of 16x16 (v_mfma_i32_16x16x64_i8, v_mfma_f32_16x16x128_f8f6f4).
// In a block a lane owns output row m = l%16 and the columns n = 4*(l/16) + {0..3}.  One
// v_permlane16_swap per word over two neighbouring blocks gives each lane 8 consecutive columns of one
// of them: lanes 0-15 block 2jp columns 0-7, lanes 16-31 block 2jp+1 columns 0-7, lanes 32-47 block
// 2jp columns 8-15, lanes 48-63 block 2jp+1 columns 8-15.
// NB: 16x16 blocks per operand and wavefront (8: 256x256 tile, 4: 128x128 tile); the tile edge is 32 * NB.
// OUTK (int8 form): element type of out and bias, DAXQ_BF16 / DAXQ_F16 / DAXQ_F32.  A template argument, i.e. a kernel
// of its own per type: with all three forms inside one kernel behind uniform branches its code grew from 27 to 44 KB
// and the bf16 launches at K = 1536, which change between main loop and epilogue every 24 slices, lost 2.7 %; with
// the choice inside the loops they lost 2 to 11 % everywhere.
template <bool DUMP, int NB = 8, bool FP8 = false, int OUTK = DAXQ_BF16>
__device__ __forceinline__ void tile256_epilogue16(const GemmArgs& p, typename Acc16<FP8>::type (&acc)[NB][NB], uint8_t* smem, int m0, int n0, int t,
                                                   int wm, int wn, int l15, int g4, float pre_sx, float pre_sw,
                                                   float pre_bias) {
    constexpr int BT = 32 * NB, WT = 16 * NB;
    float* s_sx = reinterpret_cast<float*>(smem);
    float* s_sw = s_sx + BT;
    float* s_bias = s_sw + BT;
    if (BT == 256 || t < BT) {
        s_sx[t] = pre_sx;
        s_sw[t] = pre_sw;
        s_bias[t] = pre_bias;
    }
    __syncthreads();

    if constexpr (DUMP) {
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                const int64_t m = m0 + wm * WT + i * 16 + l15;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    if constexpr (FP8) static_cast<float*>(p.acc)[m * p.ldacc + n0 + wn * WT + j * 16 + 4 * g4 + v] = acc[j][i][v];
                    else static_cast<int32_t*>(p.acc)[m * p.ldacc + n0 + wn * WT + j * 16 + 4 * g4 + v] = acc[j][i][v];
                }
            }
    }

    float sxr[NB];
    float4 swr[NB], br[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) sxr[i] = s_sx[wm * WT + i * 16 + l15];
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const int nl = wn * WT + j * 16 + 4 * g4;
        swr[j] = *reinterpret_cast<const float4*>(s_sw + nl);
        br[j] = *reinterpret_cast<const float4*>(s_bias + nl);
    }
    __builtin_amdgcn_sched_barrier(0);

    // fp32 module (int8 form): one rounding less and four-byte outputs, a lane's four columns of a block as one store
    if constexpr (!FP8 && OUTK == DAXQ_F32) {
        {
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                const float sxv = sxr[i];
                float* orow = reinterpret_cast<float*>(p.out) + (int64_t)(m0 + wm * WT + i * 16 + l15) * p.ldo + n0 + wn * WT + 4 * g4;
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    const float sws[4] = {swr[j].x, swr[j].y, swr[j].z, swr[j].w};
                    const float bs[4] = {br[j].x, br[j].y, br[j].z, br[j].w};
                    float o[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        float y = (float)acc[j][i][r];
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
    // (int8 form only) out and bias are fp16 instead of bf16
    constexpr bool f16 = !FP8 && OUTK == DAXQ_F16;
    {
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        const int ml = wm * WT + i * 16 + l15;
        const float sxv = sxr[i];
        uint16_t* orow = p.out + (int64_t)(m0 + ml) * p.ldo + n0 + wn * WT + (g4 & 1) * 16 + (g4 >> 1) * 8;
#pragma unroll
        for (int jp = 0; jp < NB / 2; ++jp) {
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
                        pk[jj][h] = pack_bf16_rne(acc[j][i][r] * sxv * sws[r] + bs[r], acc[j][i][r + 1] * sxv * sws[r + 1] + bs[r + 1]);
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

// DUMP: also write the raw accumulators to p.acc (tests); a separate instantiation so that the
// production kernel carries none of that code.
template <bool FP8, bool DUMP, bool XE5 = false>
__global__ __launch_bounds__(256) void gemm_tile256_kernel(const GemmArgs p) {
    using namespace t256;
    typedef typename AccT<FP8>::type acc_t;
    typedef typename Frag<FP8>::type frag_t;

    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    int tm, tn;
    tile_of_block(p.gm, blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    int m0 = tm * BM, n0 = tn * BN;
    m0 = m0 + BM <= p.m ? m0 : p.m - BM;
    n0 = n0 + BN <= p.n ? n0 : p.n - BN;

    // ---- HBM side: load instruction j of a thread covers tile row j*32 + t/8 and LDS chunk slot t%8,
    //      i.e. global chunk (t%8) ^ f(row).  Global address = uniform row-block base (SGPR pair) +
    //      per-lane 32-bit offset (one VGPR per operand, advanced by 128 per slice).
    const int r8 = t >> 3, slot = t & 7;
    const uint32_t chunk = (uint32_t)((slot ^ swz(r8)) << 4);
    uint32_t voff_a = (uint32_t)r8 * (uint32_t)p.lda + chunk;
    uint32_t voff_b = (uint32_t)r8 * (uint32_t)p.ldb + chunk;
    const uint8_t* abase = p.a + (int64_t)m0 * p.lda;
    const uint8_t* bbase = p.b + (int64_t)n0 * p.ldb;
    const int64_t a_step = 32 * p.lda, b_step = 32 * p.ldb;

    // ---- LDS side
    FragAddr fa;
    const int l31 = lane & 31, hi = lane >> 5;
    fa.hi = hi;
    fa.fl = swz(l31);
    fa.a_rd = smem + (wm * 128 + l31) * BK;
    fa.b_rd = smem + A_BYTES + (wn * 128 + l31) * BK;

    acc_t acc[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[j][i][v] = 0;

    const int KT = p.k / BK;
    frag_t fa0[4] = {}, fb0[4] = {}, fa1[4] = {}, fb1[4] = {};

    // MFMA steps 0 .. n-2 of a slice, each overlapped with the fragment reads of the next step
    auto steps_but_last = [&](int cur) {
        if constexpr (!FP8) {
            load_frags<FP8>(fa, cur, 1, fa1, fb1);
            mfma_step<FP8, XE5>(acc, fa0, fb0);
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                __builtin_amdgcn_sched_group_barrier(DAXQ_SG_DS_RD, 1, 0);
                __builtin_amdgcn_sched_group_barrier(DAXQ_SG_MFMA, 2, 0);
            }
            load_frags<FP8>(fa, cur, 2, fa0, fb0);
            mfma_step<FP8, XE5>(acc, fa1, fb1);
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                __builtin_amdgcn_sched_group_barrier(DAXQ_SG_DS_RD, 1, 0);
                __builtin_amdgcn_sched_group_barrier(DAXQ_SG_MFMA, 2, 0);
            }
            load_frags<FP8>(fa, cur, 3, fa1, fb1);
            mfma_step<FP8, XE5>(acc, fa0, fb0);
#pragma unroll
            for (int g = 0; g < 8; ++g) {
                __builtin_amdgcn_sched_group_barrier(DAXQ_SG_DS_RD, 1, 0);
                __builtin_amdgcn_sched_group_barrier(DAXQ_SG_MFMA, 2, 0);
            }
        } else {
            load_frags<FP8>(fa, cur, 1, fa1, fb1);
            mfma_step<FP8, XE5>(acc, fa0, fb0);
#pragma unroll
            for (int g = 0; g < 16; ++g) {
                __builtin_amdgcn_sched_group_barrier(DAXQ_SG_DS_RD, 1, 0);
                __builtin_amdgcn_sched_group_barrier(DAXQ_SG_MFMA, 1, 0);
            }
        }
    };
    auto next_frags = [&](int nxt) {
        load_frags<FP8>(fa, nxt, 0, fa0, fb0);
    };

    {
        // LDS address of a DMA load is wave-uniform (M0): 64 lanes x 16 B land in a row.
        const uint32_t lds0 = (uint32_t)(uintptr_t)(DAXQ_LDS uint8_t*)smem;
        const uint32_t wave_lds = lds0 + (uint32_t)__builtin_amdgcn_readfirstlane(wave * 1024);
        auto issue_one = [&](int stage, int g) {  // g = 0..7: A rows g*32.., g = 8..15: B rows (g-8)*32..
            if (g < 8)
                __builtin_amdgcn_global_load_lds((const DAXQ_GLOBAL void*)(abase + g * a_step + voff_a),
                                                 (DAXQ_LDS void*)(uintptr_t)(wave_lds + stage * STAGE + g * 4096), 16, 0, 0);
            else
                __builtin_amdgcn_global_load_lds((const DAXQ_GLOBAL void*)(bbase + (g - 8) * b_step + voff_b),
                                                 (DAXQ_LDS void*)(uintptr_t)(wave_lds + stage * STAGE + A_BYTES + (g - 8) * 4096), 16, 0, 0);
        };
        auto advance = [&]() {
            voff_a += BK;
            voff_b += BK;
        };
        auto issue = [&](int stage) {
#pragma unroll
            for (int g = 0; g < 16; ++g) issue_one(stage, g);
            advance();
        };
        // One K slice.  ISSUE: start the loads of slice kt+2 into the buffer slice kt leaves; NEXT:
        // prefetch the first fragments of slice kt+1.  Compile-time, so the body is one basic block.
        // The last MFMA step is cut into 16 scheduling regions of one MFMA, one DMA load and (for the
        // first 8) one fragment read each: issued as a burst, the loads back up the address unit and
        // block the in-order instruction stream, MFMAs included, behind them.
        // INT8 keeps four fragment sets, one per MFMA step of a slice, and reads them two steps ahead:
        // the HBM->LDS writes of the slice in flight share the LDS with these reads, and one step
        // (16 MFMAs) of slack did not cover the delays that causes.  The barrier sits after step 1, when
        // all fragments of the slice have been read; steps 2 and 3 then pull the next slice's first two
        // fragment sets while step 2 also issues the loads of slice kt+2.
        frag_t fa2[4] = {}, fb2[4] = {}, fa3[4] = {}, fb3[4] = {};
        auto slice = [&](int cur, auto ISSUE, auto NEXT) {
            if constexpr (FP8) {
                steps_but_last(cur);
                // slice kt+1 has landed for every wave, and every wave is done reading slice kt
                __builtin_amdgcn_s_waitcnt(vmcnt_imm(0) & lgkmcnt0_mask());
                __builtin_amdgcn_s_barrier();
#pragma unroll
                for (int g = 0; g < 16; ++g) {
                    if constexpr (ISSUE.value) issue_one(cur, g);
                    if constexpr (NEXT.value)
                        if (g < 8) load_one_frag<FP8>(fa, cur ^ 1, g, fa0, fb0);
                    mfma_one<FP8, XE5>(acc, g, fa1, fb1);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if constexpr (ISSUE.value) advance();
            } else {
                {
                    load_frags<FP8>(fa, cur, 2, fa2, fb2);
                    mfma_step<FP8, XE5>(acc, fa0, fb0);
#pragma unroll
                    for (int g = 0; g < 8; ++g) {
                        __builtin_amdgcn_sched_group_barrier(DAXQ_SG_DS_RD, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(DAXQ_SG_MFMA, 2, 0);
                    }
                    load_frags<FP8>(fa, cur, 3, fa3, fb3);
                    mfma_step<FP8, XE5>(acc, fa1, fb1);
#pragma unroll
                    for (int g = 0; g < 8; ++g) {  // reads first, so that they are over when the barrier comes
                        __builtin_amdgcn_sched_group_barrier(DAXQ_SG_DS_RD, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(DAXQ_SG_MFMA, 1, 0);
                    }
                }
                // slice kt+1 has landed for every wave, and every wave has read all of slice kt
                __builtin_amdgcn_s_waitcnt(vmcnt_imm(0) & lgkmcnt0_mask());
                __builtin_amdgcn_s_barrier();
#pragma unroll
                for (int g = 0; g < 16; ++g) {
                    if constexpr (ISSUE.value) issue_one(cur, g);
                    if constexpr (NEXT.value)
                        if (g < 8) load_one_frag<FP8>(fa, cur ^ 1, g, fa0, fb0);
                    mfma_one<FP8, XE5>(acc, g, fa2, fb2);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if constexpr (ISSUE.value) advance();
                {
                    if constexpr (NEXT.value) load_frags<FP8>(fa, cur ^ 1, 1, fa1, fb1);
                    mfma_step<FP8, XE5>(acc, fa3, fb3);
                    if constexpr (NEXT.value) {
#pragma unroll
                        for (int g = 0; g < 8; ++g) {
                            __builtin_amdgcn_sched_group_barrier(DAXQ_SG_DS_RD, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(DAXQ_SG_MFMA, 2, 0);
                        }
                    }
                }
            }
        };
        issue(0);
        if (KT > 1) {
            issue(1);
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(LOADS));  // slice 0 has landed, slice 1 may be in flight
        } else {
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        }
        __builtin_amdgcn_s_barrier();
        next_frags(0);
        if constexpr (!FP8) load_frags<FP8>(fa, 0, 1, fa1, fb1);
        int kt = 0;
        for (; kt + 2 < KT; ++kt) slice(kt & 1, Yes{}, Yes{});
        if (kt + 1 < KT) {
            slice(kt & 1, No{}, Yes{});
            ++kt;
        }
        slice(kt & 1, No{}, No{});
    }

    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    // a missing bias is + (-0.0): x + (-0.0) == x bit for bit
    tile256_epilogue<FP8, DUMP>(p, acc, smem, m0, n0, t, wm, wn, l31, hi, p.sx[m0 + t], p.sw[n0 + t],
                                p.bias ? bf16_bits_to_f32(p.bias[n0 + t]) : -0.0f);
}

// raises the kernel's dynamic LDS limit on the current device (once per device)
template <bool FP8, bool DUMP, bool XE5 = false>
static int prepare_tile256() {
    static std::atomic<uint64_t> lds_set{0};  // per instantiation
    return ensure_dynamic_lds(reinterpret_cast<const void*>(gemm_tile256_kernel<FP8, DUMP, XE5>), t256::SMEM, lds_set);
}

template <bool FP8, bool DUMP, bool XE5 = false>
static int launch_tile256_impl(const GemmArgs& a, hipStream_t st) {
    using namespace t256;
    auto kern = gemm_tile256_kernel<FP8, DUMP, XE5>;
    if (int rc = prepare_tile256<FP8, DUMP, XE5>()) return rc;
    const int64_t nt = (int64_t)a.tiles_m * a.tiles_n;
    if (nt > 0x7fffffff) return fail(DAXQ_ERR_ARG, "gemm: too many tiles");
    hipLaunchKernelGGL(kern, dim3((unsigned)nt), dim3(T), SMEM, st, a);
    return check_launch("gemm_tile256");
}

template <bool FP8>
int launch_tile256(const GemmArgs& a0, bool x_e5m2, hipStream_t st) {
    using namespace t256;
    GemmArgs a = a0;
    a.tiles_m = (a.m + BM - 1) / BM;
    a.tiles_n = (a.n + BN - 1) / BN;
    if constexpr (FP8) {
        if (x_e5m2)
            return a.acc ? launch_tile256_impl<true, true, true>(a, st) : launch_tile256_impl<true, false, true>(a, st);
    }
    return a.acc ? launch_tile256_impl<FP8, true>(a, st) : launch_tile256_impl<FP8, false>(a, st);
}

// workgroups of a launch of 256x256 tiles in the tile order a.order
static inline int64_t grid_of_order(const GemmArgs& a) {
    switch (a.order) {
        case 1: return patched_grid(a.tiles_m, a.tiles_n);
        case 2: return supergroups_grid(a.tiles_m, a.tiles_n);
        case 3: return banded_grid(a.tiles_m, a.tiles_n, 8);
        case 4: return banded_grid(a.tiles_m, a.tiles_n, 4);
        case 5: return swept_grid(a.tiles_m, a.tiles_n, 4);
        case 6: return swept_grid(a.tiles_m, a.tiles_n, 8);
        default: return (int64_t)a.tiles_m * a.tiles_n;
    }
}

// ---------------------------------------------------------------------------------------------
// Five-stage form of the same tile: K in 64-byte slices, five 32 KB LDS stages (all 160 KB).
//
// The two-stage kernel above issues the 16 loads of a 128-byte slice in a burst (one per MFMA of one
// step) and gives them between one and two MFMA steps less than a slice time to land.  Here a stage is
// half as deep, so the same LDS holds the slice being read plus four more, and the load stream is
// even: 8 loads per 64-byte slice, one every fourth (INT8) or second (FP8) MFMA.
//   * loads are issued in pairs of slices (2q, 2q+1) so that the two 64-byte halves of a 128-byte
//     line are requested by adjacent instructions (the second hits L1: measured at the full-line
//     rate, whereas half lines requested a slice apart run at half of it);
//   * the A loads of pair q+2 go out during slice 2q, its B loads during slice 2q+1; the pair has to
//     have landed at the barrier of slice 2q+3;
//   * fragments of slice s+1 are read during slice s into the other of two register sets.
// LDS layout of an operand part: [256 rows][64 B], 16-byte chunk c of row r stored at chunk
// c ^ ((r >> 2) & 3) (32x32 MFMA forms) or c ^ ((r >> 1) & 3) (16x16 form): the ds_read_b128 of either form
// then runs at the full LDS rate.
//
// BT: tile edge.  256 is the form described above; 128 (wavefronts of 64 x 64, five 16 KB stages, two workgroups
// per CU) is the same pipeline for launches with too few 256-tiles to fill the CUs.
namespace t5 {
constexpr int BKS = 64, NST = 5, T = 256;
}  // namespace t5

// accumulators of a wavefront's 128 x 128 outputs
template <bool FP8, bool N16>
struct TileAcc {
    typedef typename AccT<FP8>::type type;  // 32x32 blocks
};
template <>
struct TileAcc<false, true> {
    typedef v4i type;  // 16x16 blocks
};

// N16 (INT8 only): the slice is one v_mfma_i32_16x16x64_i8 per 16x16 block (64 per wave and slice) instead
// of two v_mfma_i32_32x32x32_i8 per 32x32 block (32).  Same LDS bytes, fragment registers and MFMA
// cycles; the narrow shape moves fewer accumulator bytes per operation and sustains a higher clock
// under the board's power limit.
//
// SPLITK (128 tile): K is cut into p.splits ranges and blockIdx.x = tile * splits + split.  A workgroup accumulates
// its range, writes the accumulators to the workspace (one 16-byte vector per lane and store instruction), and
// counts itself in at the tile's counter; the workgroup that arrives last adds the partial results of all ranges
// in range order (so FP8 sums do not depend on who was last) and runs the epilogue.  No workgroup waits for
// another.  The last one sets the counter back to zero.
template <bool FP8, bool DUMP, int F8, bool N16 = false, int BT = 256, bool SPLITK = false, int D = 2, int OUTK = DAXQ_BF16>
__global__ __launch_bounds__(256) void gemm_tile256s5_kernel(const GemmArgs p) {
    static_assert(OUTK == DAXQ_BF16 || (N16 && !SPLITK && !DUMP), "fp16 / fp32 outputs exist in the 16x16 int8 form");
    using namespace t5;
    static_assert(!(FP8 && N16), "the 16x16 form exists for INT8 only");
    static_assert(BT == 256 || BT == 128, "tile edge");
    static_assert(D == 2 || (D == 4 && BT == 128 && !SPLITK), "the deep ring exists on 128 tiles (nine 16 KB stages)");
    constexpr int NSTG = 2 * D + 1;                   // LDS stages: the slice being read plus D pairs in flight
    typedef typename Frag<FP8>::type frag_t;
    constexpr int WT = BT / 2;                        // edge of a wavefront's outputs
    constexpr int NB = WT / (N16 ? 16 : 32);          // MFMA blocks per operand and wavefront: 8 / 4 (256), 4 / 2 (128)
    constexpr int A_BYTES = BT * BKS, STAGE = 2 * A_BYTES;
    constexpr int PAIR_LOADS = BT / 16;               // DMA loads per thread and pair of slices
    constexpr int JB = BT / 64;                       // 64-row blocks of an operand part (one DMA instruction each)
    constexpr int STEPS = FP8 ? 1 : 2;               // MFMA steps per 64-byte slice (32x32 form)
    constexpr int NREG = N16 ? NB * NB : NB * NB * STEPS;  // MFMAs = scheduling regions per slice
    constexpr int DMA_EVERY = NREG / (PAIR_LOADS / 2);     // regions per DMA load
    constexpr int READ_EVERY = NREG >= 48 ? 3 : NREG / (2 * NB);  // N16: regions per fragment read (2 * NB reads)

    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    int tm, tn;
    int tile_id = blockIdx.x, split = 0, klen = p.k;  // klen: bytes of K this workgroup covers, a multiple of 128
    if constexpr (SPLITK) {
        static_assert(BT == 128 && !DUMP, "split-K exists on 128 tiles, without the accumulator dump");
        tile_id = blockIdx.x / p.splits;
        split = blockIdx.x - tile_id * p.splits;
        klen = p.k / p.splits;
    }
    if (!SPLITK && p.order == 1) {
        if (!tile_of_block_patched(tile_id, p.tiles_m, p.tiles_n, tm, tn)) return;  // padding slot (before any barrier)
    } else if (!SPLITK && p.order == 2) {
        if (!tile_of_block_supergroups(tile_id, p.tiles_m, p.tiles_n, tm, tn)) return;
    } else if (!SPLITK && p.order >= 5) {
        if (!tile_of_block_swept(tile_id, p.tiles_m, p.tiles_n, p.order == 5 ? 4 : 8, tm, tn)) return;
    } else if (!SPLITK && p.order >= 3) {
        if (!tile_of_block_banded(tile_id, p.tiles_m, p.tiles_n, p.order == 3 ? 8 : 4, tm, tn)) return;
    } else if (BT == 128 && !SPLITK && p.quad_base) {
        tile_of_block(p.gm, p.quad_base - 1 + (tile_id >> 2), p.tiles_m, p.tiles_n, tm, tn);  // the 256x256 tile
    } else {
        tile_of_block(p.gm, tile_id, p.tiles_m, p.tiles_n, tm, tn);
    }
    int m0 = tm * BT, n0 = tn * BT;
    m0 = m0 + BT <= p.m ? m0 : p.m - BT;
    n0 = n0 + BT <= p.n ? n0 : p.n - BT;
    if (BT == 128 && !SPLITK && p.quad_base) {  // quadrant tile_id % 4 of the 256x256 tile, whose origin is shifted inwards at the edges
        m0 = tm * 256, n0 = tn * 256;
        m0 = (m0 + 256 <= p.m ? m0 : p.m - 256) + ((tile_id >> 1) & 1) * 128;
        n0 = (n0 + 256 <= p.n ? n0 : p.n - 256) + (tile_id & 1) * 128;
    }

    // ---- HBM side.  One wave instruction fills 1 KB of LDS = 16 rows x 64 B: lane l -> row l/4,
    //      stored chunk l%4, i.e. global chunk (l%4) ^ ((row>>2)&3).  Instruction j of a thread
    //      covers tile rows j*64 + t/4.
    //      N16 swizzles with (row>>1)&3 instead: its fragment reads (16 rows x 4 chunks per instruction) are
    //      conflict free with that one and lose a fifth of the LDS rate with (row>>2)&3 (measured).
    const uint32_t gsw = (uint32_t)(((t & 3) ^ ((N16 ? t >> 3 : t >> 4) & 3)) << 4);
    uint32_t voff_a = (uint32_t)(t >> 2) * (uint32_t)p.lda + gsw;
    uint32_t voff_b = (uint32_t)(t >> 2) * (uint32_t)p.ldb + gsw;
    uint32_t voff_a1 = voff_a + BKS, voff_b1 = voff_b + BKS;  // second half of the 128-byte line
    const uint8_t* abase = p.a + (int64_t)m0 * p.lda + (int64_t)split * klen;
    const uint8_t* bbase = p.b + (int64_t)n0 * p.ldb + (int64_t)split * klen;
    const int64_t a_step = 64 * p.lda, b_step = 64 * p.ldb;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(DAXQ_LDS uint8_t*)smem;
    const uint32_t wave_lds = lds0 + (uint32_t)__builtin_amdgcn_readfirstlane(wave * 1024);
    // load g of a pair (16 for a 256 tile): first half of them operand A, row block (g/2) % JB, half g%2 -> stage o0 / o1.
    // Address = uniform row-block base (SGPR pair) + per-lane 32-bit offset: no VALU work per load.
    auto issue_one = [&](uint32_t o0, uint32_t o1, int g) {
        const int opnd = g / (PAIR_LOADS / 2), j = (g >> 1) % JB, half = g & 1;
        const uint8_t* src = opnd ? bbase + j * b_step : abase + j * a_step;
        const uint32_t voff = opnd ? (half ? voff_b1 : voff_b) : (half ? voff_a1 : voff_a);
        const uint32_t dst = wave_lds + (half ? o1 : o0) + opnd * A_BYTES + j * 4096;
        __builtin_amdgcn_global_load_lds((const DAXQ_GLOBAL void*)(src + voff), (DAXQ_LDS void*)(uintptr_t)dst, 16, 0, 0);
    };
    auto advance_a = [&]() {
        voff_a += 2 * BKS;
        voff_a1 += 2 * BKS;
    };
    auto advance_b = [&]() {
        voff_b += 2 * BKS;
        voff_b1 += 2 * BKS;
    };
    auto advance = [&]() {
        advance_a();
        advance_b();
    };

    // ---- LDS side: row (w*128 + i*32 + l%32), chunk c of the slice at (c ^ g) * 16, g = (l%32 >> 2) & 3
    //      N16: row (w*128 + i*16 + l%16), the lane's K chunk is l/16
    const int l31 = lane & 31, hi = lane >> 5;
    const int lr = N16 ? (lane & 15) : l31;  // row of the lane inside an MFMA block
    const int gq = ((N16 ? lr >> 1 : lr >> 2)) & 3;
    const uint8_t* a_rd = smem + (wm * WT + lr) * BKS;
    const uint8_t* b_rd = smem + A_BYTES + (wn * WT + lr) * BKS;
    // one fragment: f = 0..3 A block f, 4..7 B block f-4; step ks of the slice in the stage at offset o
    // (N16: ks selects the upper four of the eight 16-row blocks; every fragment spans the whole slice)
    auto read_frag = [&](uint32_t o, int ks, int f, frag_t (&af)[4], frag_t (&bf)[4]) {
        if constexpr (N16) {
            const uint8_t* pr = (f < 4 ? a_rd : b_rd) + o + (ks * 4 + (f & 3)) * 16 * BKS;
            (f < 4 ? af[f & 3] : bf[f & 3]) = *reinterpret_cast<const v4i*>(pr + (((lane >> 4) ^ gq) << 4));
            return;
        }
        if ((f & 3) >= NB) return;  // 128 tile: two 32-row blocks per operand
        const uint8_t* pr = (f < 4 ? a_rd : b_rd) + o + (f & 3) * 32 * BKS;
        if constexpr (!FP8) {
            const int xo = ((ks * 2 + hi) ^ gq) << 4;
            (f < 4 ? af[f & 3] : bf[f & 3]) = *reinterpret_cast<const v4i*>(pr + xo);
        } else {
            const int xo0 = ((hi * 2) ^ gq) << 4, xo1 = ((hi * 2 + 1) ^ gq) << 4;
            v4i lo = *reinterpret_cast<const v4i*>(pr + xo0);
            v4i up = *reinterpret_cast<const v4i*>(pr + xo1);
            (f < 4 ? af[f & 3] : bf[f & 3]) = __builtin_shufflevector(lo, up, 0, 1, 2, 3, 4, 5, 6, 7);
        }
    };

    typename TileAcc<FP8, N16>::type acc[NB][NB];

    // fragment sets: [slice parity][MFMA step] (N16: [slice parity][blocks 0-3 / 4-7])
    frag_t fa00[4] = {}, fb00[4] = {}, fa01[4] = {}, fb01[4] = {}, fa10[4] = {}, fb10[4] = {}, fa11[4] = {}, fb11[4] = {};

    const int S = klen / BKS;  // slices; even because K (and each split range) is a multiple of 128
    // stage offsets of slices s .. s+2D-1 and, last, of slice s-1 (s = the even slice of the current pair)
    uint32_t st[NSTG];
#pragma unroll
    for (int i = 0; i < NSTG; ++i) st[i] = i * STAGE;

    // One slice.  ODD: slice parity (which register set is consumed).  At its barrier slice s+1 has
    // landed for every wave and every wave has the fragments of slice s in registers.
    //   ISSUE  start half of pair (s+2D, s+2D+1) (s even: the A loads; s odd: the B loads of the same
    //          pair) into the stages o_ld0 / o_ld1 that slices s-1 and s have left
    //   NEXT   slice s+1 exists: read its fragments into the other set
    //   YOUNG  number of loads issued after those of slice s+1 that may stay in flight: D-1 whole pairs at
    //          an even slice, D-2 pairs and the A half of the newest pair at an odd one (vmcnt retires in order)
    //   EXTRA  younger loads that are not tile loads (the epilogue's scales) and may stay in flight
    //   FIRST  slice 0 of the tile: its MFMAs start from zero, the accumulators need no clearing
    auto slice = [&](auto ODD, auto ISSUE, auto NEXT, auto YOUNG, auto EXTRA, auto FIRST, uint32_t o_next, uint32_t o_ld0, uint32_t o_ld1)
                     __attribute__((always_inline)) {
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(YOUNG.value + EXTRA.value) & lgkmcnt0_mask());
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int g = 0; g < NREG; ++g) {
            if constexpr (ISSUE.value) {
                if (g % DMA_EVERY == 0) issue_one(o_ld0, o_ld1, g / DMA_EVERY + (ODD.value ? PAIR_LOADS / 2 : 0));
            }
            if constexpr (NEXT.value && N16) {  // 2 * NB reads, one every READ_EVERY regions
                if (g % READ_EVERY == 0 && g / READ_EVERY < 2 * NB) {
                    // NB = 8: blocks 0-3 of A and B, then blocks 4-7; NB = 4: blocks 0-3 of A and B
                    const int idx = NB == 8 ? g / READ_EVERY : (g / READ_EVERY < NB ? g / READ_EVERY : 4 + g / READ_EVERY - NB);
                    if constexpr (ODD.value) {
                        if (idx < 8) read_frag(o_next, 0, idx, fa00, fb00);
                        else read_frag(o_next, 1, idx - 8, fa01, fb01);
                    } else {
                        if (idx < 8) read_frag(o_next, 0, idx, fa10, fb10);
                        else read_frag(o_next, 1, idx - 8, fa11, fb11);
                    }
                }
            } else if constexpr (NEXT.value) {
                // fragment fi of a step: the NB blocks of A, then the NB blocks of B (slot 4 + block in read_frag)
                if constexpr (!FP8) {  // 2 * NB reads of step 0 in the first regions, then those of step 1
                    if (g < 4 * NB) {
                        const int fi = g % (2 * NB), f = fi < NB ? fi : 4 + fi - NB;
                        if (g < 2 * NB) {
                            if constexpr (ODD.value) read_frag(o_next, 0, f, fa00, fb00);
                            else read_frag(o_next, 0, f, fa10, fb10);
                        } else {
                            if constexpr (ODD.value) read_frag(o_next, 1, f, fa01, fb01);
                            else read_frag(o_next, 1, f, fa11, fb11);
                        }
                    }
                } else {
                    if (g < 2 * NB) {
                        const int f = g < NB ? g : 4 + g - NB;
                        if constexpr (ODD.value) read_frag(o_next, 0, f, fa00, fb00);
                        else read_frag(o_next, 0, f, fa10, fb10);
                    }
                }
            }
            if constexpr (N16) {
                const int j = g / NB, i = g % NB;  // B block j, A block i
                const v4i bfr = ODD.value ? (j < 4 ? fb10[j & 3] : fb11[j & 3]) : (j < 4 ? fb00[j & 3] : fb01[j & 3]);
                const v4i afr = ODD.value ? (i < 4 ? fa10[i & 3] : fa11[i & 3]) : (i < 4 ? fa00[i & 3] : fa01[i & 3]);
                // accumulator tied in place in AGPRs: left to the register allocator, the 64 four-register
                // accumulators rotate through one another with copies in the loop
                if constexpr (FIRST.value)
                    asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, 0" : "=a"(acc[j][i]) : "v"(bfr), "v"(afr));
                else
                    asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(acc[j][i]) : "v"(bfr), "v"(afr));
            } else if constexpr (!FP8) {
                if constexpr (ODD.value) {
                    if (g < NB * NB) mfma_one<FP8, F8, false, NB>(acc, g, fa10, fb10);
                    else mfma_one<FP8, F8, false, NB>(acc, g - NB * NB, fa11, fb11);
                } else {
                    if (g < NB * NB) mfma_one<FP8, F8, FIRST.value, NB>(acc, g, fa00, fb00);
                    else mfma_one<FP8, F8, false, NB>(acc, g - NB * NB, fa01, fb01);
                }
            } else {
                if constexpr (ODD.value) mfma_one<FP8, F8, false, NB>(acc, g, fa10, fb10);
                else mfma_one<FP8, F8, FIRST.value, NB>(acc, g, fa00, fb00);
            }
            // loop bookkeeping inside the last regions, in the issue slots an MFMA leaves free, instead of
            // in a block of its own behind the slice: lane offsets of the operand this slice loaded, and
            // (odd slice) the rotation of the stage offsets by one pair
            if constexpr (ISSUE.value) {
                // behind the slice's last load (with a load in every region that is the last region)
                if (g == (DMA_EVERY == 1 ? NREG - 1 : NREG - 2)) {
                    if constexpr (ODD.value) advance_b();
                    else advance_a();
                }
            }
            if constexpr (ODD.value) {
                if (g == NREG - 1) {
                    const uint32_t r0 = st[0], r1 = st[1];
#pragma unroll
                    for (int i = 0; i + 2 < NSTG; ++i) st[i] = st[i + 2];
                    st[NSTG - 2] = r0;
                    st[NSTG - 1] = r1;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // a pair of slices (s, s+1), s even.  The stage offsets are passed by value: the odd slice rotates them in its
    // last region.
    auto pair = [&](auto ISSUE, auto YOUNG_E, auto YOUNG_O, auto NEXT_O, auto EXTRA, auto FIRST) __attribute__((always_inline)) {
        slice(No{}, ISSUE, Yes{}, YOUNG_E, EXTRA, FIRST, st[1], st[NSTG - 1], st[0]);
        slice(Yes{}, ISSUE, NEXT_O, YOUNG_O, EXTRA, No{}, st[2], st[NSTG - 1], st[0]);
    };
    // a pair of the steady state (it starts pair q+D), and tail pair TL of the D pairs behind the last loads
    typedef Int<(D - 1) * PAIR_LOADS> SteadyE;
    typedef Int<(D - 2) * PAIR_LOADS + PAIR_LOADS / 2> SteadyO;
    auto tail_pair = [&](auto TL) __attribute__((always_inline)) {
        constexpr int t = decltype(TL)::value;
        pair(No{}, Int<(D - 1 - t) * PAIR_LOADS>{}, Int<(D - 2 - t > 0 ? D - 2 - t : 0) * PAIR_LOADS>{}, Int<(t < D - 1)>{}, Int<3>{}, No{});
    };

    // ---- prologue: pairs 0 .. D-1 in flight, pair 0 landed, fragments of slice 0 in set 0
#pragma unroll
    for (int g = 0; g < PAIR_LOADS; ++g) issue_one(0, STAGE, g);
    advance();
    if constexpr (D == 2) {
        if (S >= 4) {
#pragma unroll
            for (int g = 0; g < PAIR_LOADS; ++g) issue_one(2 * STAGE, 3 * STAGE, g);
            advance();
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(PAIR_LOADS));
        } else {
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        }
    } else {  // the launcher sends only K of at least 2 D pairs here
#pragma unroll
        for (int d = 1; d < D; ++d) {
#pragma unroll
            for (int g = 0; g < PAIR_LOADS; ++g) issue_one(2 * d * STAGE, (2 * d + 1) * STAGE, g);
            advance();
        }
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((D - 1) * PAIR_LOADS));
    }
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int f = 0; f < 8; ++f) {
        read_frag(0, 0, f, fa00, fb00);
        if constexpr (!FP8 && !(N16 && NB == 4)) read_frag(0, 1, f, fa01, fb01);  // 16x16 form: blocks 4-7 exist for NB = 8
    }

    const int Q = S >> 1;  // pairs
    if (D > 2 || Q >= 3) {
        pair(Yes{}, SteadyE{}, SteadyO{}, Yes{}, Int<0>{}, Yes{});
    } else {  // short K: no pair to peel, clear the accumulators instead
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int i = 0; i < NB; ++i) acc[j][i] = typename TileAcc<FP8, N16>::type{};
    }
    for (int q = 1; q + D < Q; ++q) pair(Yes{}, SteadyE{}, SteadyO{}, Yes{}, Int<0>{}, No{});

    // The epilogue's scales and bias are requested here, behind the last tile loads, so that their
    // latency is covered by the remaining two pairs of slices.  Always three loads (a missing bias
    // reads a scale instead and is replaced by -0.0: x + (-0.0) == x bit for bit).
    // (every wavefront issues them, so that the counts the waits are written for hold: with a 128 tile the upper
    // two wavefronts repeat the loads of the lower two and drop the values)
    const int tt = t & (BT - 1);
    const float pre_sx = p.sx[m0 + tt], pre_sw = p.sw[n0 + tt];
    uint32_t pre_b;  // the bias element's bits: bf16 / fp16, or fp32
    if constexpr (OUTK == DAXQ_F32) pre_b = __float_as_uint((p.bias ? reinterpret_cast<const float*>(p.bias) : p.sw)[n0 + tt]);
    else pre_b = (p.bias ? p.bias : reinterpret_cast<const uint16_t*>(p.sw))[n0 + tt];
    __builtin_amdgcn_sched_barrier(0);

    if constexpr (D == 2) {
        if (Q >= 2) tail_pair(Int<0>{});
        tail_pair(Int<1>{});
    } else {
        tail_pair(Int<0>{});
        tail_pair(Int<1>{});
        tail_pair(Int<2>{});
        tail_pair(Int<3>{});
    }

    if constexpr (N16) {
        // The 16x16 MFMAs are inline asm, so the compiler cannot count the wait states between one of them and a
        // VALU read of its result, and it places such reads right behind the MFMA if nothing stops it.  Volatile
        // asm statements keep their order: 24 idle cycles first, then every accumulator is passed through an empty
        // statement, which no read of it can move above.
        asm volatile("s_nop 15\n\ts_nop 7");
#pragma unroll
        for (int j = 0; j < NB; j += 2) {
            if constexpr (NB == 8) {
                asm volatile(""
                             : "+a"(acc[j][0]), "+a"(acc[j][1]), "+a"(acc[j][2]), "+a"(acc[j][3]), "+a"(acc[j][4]), "+a"(acc[j][5]),
                               "+a"(acc[j][6]), "+a"(acc[j][7]), "+a"(acc[j + 1][0]), "+a"(acc[j + 1][1]), "+a"(acc[j + 1][2]),
                               "+a"(acc[j + 1][3]), "+a"(acc[j + 1][4]), "+a"(acc[j + 1][5]), "+a"(acc[j + 1][6]), "+a"(acc[j + 1][7]));
            } else {
                asm volatile(""
                             : "+a"(acc[j][0]), "+a"(acc[j][1]), "+a"(acc[j][2]), "+a"(acc[j][3]), "+a"(acc[j + 1][0]),
                               "+a"(acc[j + 1][1]), "+a"(acc[j + 1][2]), "+a"(acc[j + 1][3]));
            }
        }
    }
    if constexpr (SPLITK) {
        // ---- partial accumulators -> workspace; the last workgroup of the tile sums all of them.
        // Partial results cross from one XCD's L2 to another's.  A device-wide fence would do that by writing back
        // and invalidating the whole L2 of the XCD, once per wavefront (measured: 0.3 us per workgroup, serialised,
        // 4x the time of the plain launch).  Instead every access to the workspace is itself an agent-scope relaxed
        // atomic (a store / load with the device-coherent cache policy), the stores are waited for (vmcnt) before the
        // workgroup's barrier, and only then does one thread count the workgroup in; the last arriver reads behind
        // a barrier that follows its own count.
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // the scale / bias loads have landed: the waits above count them
        constexpr int VPB = N16 ? 1 : 4;           // 16-byte vectors per lane and MFMA block
        constexpr int NV = NB * NB * VPB;          // per lane: 16 of them = 64 registers either way
        typedef uint64_t u64x2 __attribute__((ext_vector_type(2)));
        uint64_t* mine = static_cast<uint64_t*>(p.partials) + ((int64_t)blockIdx.x * NV * 256 + t) * 2;
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int i = 0; i < NB; ++i)
#pragma unroll
                for (int v = 0; v < VPB; ++v) {
                    v4i w;
                    if constexpr (N16) {
                        w = acc[j][i];
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) w[e] = __float_as_int(acc[j][i][4 * v + e]);  // (a by-value call: __builtin_bit_cast of a vector element reads element 0)
                    }
                    const u64x2 w2 = __builtin_bit_cast(u64x2, w);
                    uint64_t* dst = mine + (int64_t)((j * NB + i) * VPB + v) * 512;
                    __hip_atomic_store(dst, w2[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(dst + 1, w2[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // this lane's partial results have reached device-coherent memory
        __syncthreads();                           // ... and every lane's
        int* flag = reinterpret_cast<int*>(smem + 2048);  // LDS is free: nobody reads a stage after the last barrier
        if (t == 0) *flag = __hip_atomic_fetch_add(p.counters + tile_id, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == p.splits - 1;
        __syncthreads();
        if (!*flag) return;
        const uint64_t* all = static_cast<const uint64_t*>(p.partials) + ((int64_t)tile_id * p.splits * NV * 256 + t) * 2;
        // one range at a time, in range order (FP8 sums then do not depend on who came last); all loads of a range
        // are in flight together, so a range costs one trip to memory, not one per vector
        v4i sum[NV];
        for (int sp = 0; sp < p.splits; ++sp) {
            const uint64_t* src = all + (int64_t)sp * NV * 512;
            u64x2 w2[NV];
#pragma unroll
            for (int x = 0; x < NV; ++x) {
                w2[x][0] = __hip_atomic_load(src + x * 512, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                w2[x][1] = __hip_atomic_load(src + x * 512 + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
#pragma unroll
            for (int x = 0; x < NV; ++x) {
                const v4i w = __builtin_bit_cast(v4i, w2[x]);
                if (sp == 0) {
                    sum[x] = w;  // (0.0f + x would turn a -0.0 partial sum into +0.0)
                } else if constexpr (FP8) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) sum[x][e] = __float_as_int(__int_as_float(sum[x][e]) + __int_as_float(w[e]));
                } else {
                    sum[x] += w;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int i = 0; i < NB; ++i)
#pragma unroll
                for (int v = 0; v < VPB; ++v) {
                    const v4i sv = sum[(j * NB + i) * VPB + v];
                    if constexpr (N16) {
                        acc[j][i] = sv;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[j][i][4 * v + e] = __int_as_float(sv[e]);
                    }
                }
        if (t == 0) p.counters[tile_id] = 0;  // ready for the next launch on this workspace
        __syncthreads();                      // every thread has read the flag before the epilogue reuses the LDS
    }
    if constexpr (N16)
        tile256_epilogue16<DUMP, NB, false, OUTK>(p, acc, smem, m0, n0, t, wm, wn, lr, lane >> 4, pre_sx, pre_sw,
                                                  !p.bias ? -0.0f : OUTK == DAXQ_F32 ? __uint_as_float(pre_b) : OUTK == DAXQ_F16 ? f16_bits_to_f32((uint16_t)pre_b) : bf16_bits_to_f32(pre_b));
    else
        tile256_epilogue<FP8, DUMP, NB>(p, acc, smem, m0, n0, t, wm, wn, l31, hi, pre_sx, pre_sw,
                                        p.bias ? bf16_bits_to_f32(pre_b) : -0.0f);
}

// ---------------------------------------------------------------------------------------------
// FP8 on v_mfma_f32_16x16x128_f8f6f4: the 256x256 tile with 8 x 8 blocks of 16x16 per wavefront.
//
// The narrow FP8 MFMA draws less power per operation than the 32x32x64 form (register-only loops on this
// workload's values: 4.41 against 4.02 P-op/s), as the 16x16x64 form does for INT8.  Its K is 128 bytes, a PAIR of
// 64-byte slices, and the operand fragments of a pair fill 128 registers, so they cannot all be held twice beside
// 256 accumulators.  Register plan (8 registers per fragment: 16 bytes of either slice of the pair):
//   A (activation rows, MFMA "B" operand)  two sets of 8 fragments, the next pair's set read during the odd half
//   B (weight rows, MFMA "A" operand)      ONE set: the MFMAs run B block by B block (j outer, A block i inner), block
//                                          j is dead after its 8 MFMAs and is refilled in place for the next pair
//                                          right behind them; block 7, which is in use until the pair ends, has a
//                                          second register set
// LDS: five 32 KB parts, each ONE operand of ONE pair, [slice of the pair][256 rows][64 B] with the 16-byte chunk
// swizzle of the 16x16 INT8 form (chunk ^ ((row >> 1) & 3): a fragment read takes 16 rows x 4 chunks).  They form a
// ring in the order the loads are issued, ... B(q+1), A(q+1), B(q+2), A(q+2), B(q+3) ...:
//   pair q, even half   MFMAs of B blocks 0-3; DMA loads of A(q+2) into the part B(q) has left; reads B block 7 and
//                       blocks 0-2 of pair q+1
//   pair q, odd half    MFMAs of B blocks 4-7; DMA loads of B(q+3) into the part A(q) has left; reads B blocks 3-6
//                       and all of A of pair q+1
// One barrier per half: at the first B(q+1) has landed, at the second A(q+1); every load has two to three slice
// times to land, as in the 64-byte-slice kernels above, and the half-line pairing of the loads is the same.
// A and B of a lane hold the same K bytes (chunk l/16 of the pair's first slice, then of its second), which is all
// the MFMA needs: the order of K inside an instruction is free as long as both operands agree.
namespace f16 {
constexpr int BT = 256, BKS = 64, T = 256, NPART = 5;
constexpr int HALF = BT * BKS;   // one slice of one operand: 16 KB
constexpr int PART = 2 * HALF;   // one operand of one pair: 32 KB
constexpr int SMEM = NPART * PART;
#ifndef DAXQ_F16_RD_LAG
#define DAXQ_F16_RD_LAG 0
#endif
constexpr int RD_LAG = DAXQ_F16_RD_LAG;  // regions between the last MFMA that reads a B fragment and the LDS read that refills it
constexpr int TRAIL_READS = 0;  // ds_read_b128 issued behind the last B read of a pair (block 6 at region 56)
}  // namespace f16

template <bool DUMP, int F8>
__global__ __launch_bounds__(256) void gemm_tile256f16_kernel(const GemmArgs p) {
    using namespace f16;
    constexpr int NB = 8;
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    int tm, tn;
    if (p.order == 1) {
        if (!tile_of_block_patched(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn)) return;  // padding slot (before any barrier)
    } else if (p.order == 2) {
        if (!tile_of_block_supergroups(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn)) return;
    } else if (p.order >= 5) {
        if (!tile_of_block_swept(blockIdx.x, p.tiles_m, p.tiles_n, p.order == 5 ? 4 : 8, tm, tn)) return;
    } else if (p.order >= 3) {
        if (!tile_of_block_banded(blockIdx.x, p.tiles_m, p.tiles_n, p.order == 3 ? 8 : 4, tm, tn)) return;
    } else {
        tile_of_block(p.gm, blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    }
    int m0 = tm * BT, n0 = tn * BT;
    m0 = m0 + BT <= p.m ? m0 : p.m - BT;
    n0 = n0 + BT <= p.n ? n0 : p.n - BT;

    // ---- HBM side: one wave instruction fills 1 KB of LDS = 16 rows x 64 B; lane l -> row l/4, stored chunk l%4,
    //      i.e. global chunk (l%4) ^ ((row >> 1) & 3).  Load g of an operand and pair: row block g/2 (64 rows, of which
    //      this wave fills 16), slice g%2 of the pair (the two halves of a 128-byte line, adjacent instructions).
    const uint32_t gsw = (uint32_t)(((t & 3) ^ ((t >> 3) & 3)) << 4);
    uint32_t voff_a = (uint32_t)(t >> 2) * (uint32_t)p.lda + gsw;
    uint32_t voff_b = (uint32_t)(t >> 2) * (uint32_t)p.ldb + gsw;
    uint32_t voff_a1 = voff_a + BKS, voff_b1 = voff_b + BKS;
    const uint8_t* abase = p.a + (int64_t)m0 * p.lda;
    const uint8_t* bbase = p.b + (int64_t)n0 * p.ldb;
    const int64_t a_step = 64 * p.lda, b_step = 64 * p.ldb;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(DAXQ_LDS uint8_t*)smem;
    const uint32_t wave_lds = lds0 + (uint32_t)__builtin_amdgcn_readfirstlane(wave * 1024);
    auto issue_a = [&](uint32_t part, int g) {
        const int j = g >> 1, half = g & 1;
        const uint32_t dst = wave_lds + part + half * HALF + j * 4096;
        __builtin_amdgcn_global_load_lds((const DAXQ_GLOBAL void*)(abase + j * a_step + (half ? voff_a1 : voff_a)),
                                         (DAXQ_LDS void*)(uintptr_t)dst, 16, 0, 0);
    };
    auto issue_b = [&](uint32_t part, int g) {
        const int j = g >> 1, half = g & 1;
        const uint32_t dst = wave_lds + part + half * HALF + j * 4096;
        __builtin_amdgcn_global_load_lds((const DAXQ_GLOBAL void*)(bbase + j * b_step + (half ? voff_b1 : voff_b)),
                                         (DAXQ_LDS void*)(uintptr_t)dst, 16, 0, 0);
    };
    auto advance_a = [&]() {
        voff_a += 2 * BKS;
        voff_a1 += 2 * BKS;
    };
    auto advance_b = [&]() {
        voff_b += 2 * BKS;
        voff_b1 += 2 * BKS;
    };

    // ---- LDS side: row (w*128 + i*16 + l%16), K chunk l/16 of either slice, stored at chunk (l/16) ^ ((l%16 >> 1) & 3)
    const int lr = lane & 15, kg = lane >> 4;
    const int xo = (kg ^ ((lr >> 1) & 3)) << 4;
    const uint8_t* a_rd = smem + (wm * 128 + lr) * BKS + xo;
    const uint8_t* b_rd = smem + (wn * 128 + lr) * BKS + xo;
    // A fragment is refilled as two updates of half of its registers: the register allocator then keeps the
    // fragment where it is (a fresh 8-register value per refill made it rotate the fragment sets through one
    // another with copies and spills).
    auto read_into = [&](v8i& dst, const uint8_t* base, uint32_t part, int blk) __attribute__((always_inline)) {
        const uint8_t* pr = base + part + blk * 16 * BKS;
        const v4i lo = *reinterpret_cast<const v4i*>(pr);
        const v4i up = *reinterpret_cast<const v4i*>(pr + HALF);
        const v8i lo8 = __builtin_shufflevector(lo, lo, 0, 1, 2, 3, -1, -1, -1, -1);  // (widened; the upper lanes are never taken)
        const v8i up8 = __builtin_shufflevector(up, up, 0, 1, 2, 3, -1, -1, -1, -1);
        dst = __builtin_shufflevector(lo8, dst, 0, 1, 2, 3, 12, 13, 14, 15);
        dst = __builtin_shufflevector(dst, up8, 0, 1, 2, 3, 8, 9, 10, 11);
    };

    v4f acc[NB][NB];
    // (left uninitialised on purpose: every register of a fragment is written by its first refill, and an
    // initial value would have to be kept alive, and spilled, through the prologue)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wuninitialized"
#pragma clang diagnostic ignored "-Wsometimes-uninitialized"
    v8i fa0[NB], fa1[NB];  // A fragments of even / odd pairs
    v8i fb[NB - 1];        // B fragments 0-6, refilled in place
    v8i fb7_0, fb7_1;      // B fragment 7 of even / odd pairs
#pragma clang diagnostic pop

    const int Q = p.k / (2 * BKS);  // pairs; K is a multiple of 128
    // the ring, oldest part first: at the start of pair q it holds B(q), A(q) (both read already), B(q+1), A(q+1), B(q+2)
    uint32_t r0 = 0, r1 = PART, r2 = 2 * PART, r3 = 3 * PART, r4 = 4 * PART;

    // One pair of slices.  PAR: parity of the pair (which A set and which B-7 set it consumes).
    //   ISSUE_A  pair q+2 exists: its A loads go out during the even half
    //   ISSUE_B  pair q+3 exists: its B loads go out during the odd half
    //   NEXT     pair q+1 exists: read its fragments
    //   EXTRA    younger loads that are not tile loads (the epilogue's scales) and may stay in flight
    //   FIRST    pair 0 of the tile: every block's MFMA starts from zero
    auto pair = [&](auto PAR, auto ISSUE_A, auto ISSUE_B, auto NEXT, auto EXTRA, auto FIRST) __attribute__((always_inline)) {
        constexpr bool par = PAR.value, nxt = NEXT.value;
        auto mfma = [&](int g) __attribute__((always_inline)) {
            const int j = g >> 3, i = g & 7;
            const v8i bfr = j == 7 ? (par ? fb7_1 : fb7_0) : fb[j < 7 ? j : 0];
            const v8i afr = par ? fa1[i] : fa0[i];
            // weights are the MFMA "A" operand (format select cbsz), activations the "B" operand (blgp); accumulators
            // tied in place in AGPRs
            if constexpr (FIRST.value) {
                if constexpr (F8 == 0) asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0" : "=a"(acc[j][i]) : "v"(bfr), "v"(afr));
                else if constexpr (F8 == kF8XE5) asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0 blgp:1" : "=a"(acc[j][i]) : "v"(bfr), "v"(afr));
                else if constexpr (F8 == kF8WE5) asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0 cbsz:1" : "=a"(acc[j][i]) : "v"(bfr), "v"(afr));
                else asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0 cbsz:1 blgp:1" : "=a"(acc[j][i]) : "v"(bfr), "v"(afr));
            } else {
                if constexpr (F8 == 0) asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(acc[j][i]) : "v"(bfr), "v"(afr));
                else if constexpr (F8 == kF8XE5) asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0 blgp:1" : "+a"(acc[j][i]) : "v"(bfr), "v"(afr));
                else if constexpr (F8 == kF8WE5) asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0 cbsz:1" : "+a"(acc[j][i]) : "v"(bfr), "v"(afr));
                else asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0 cbsz:1 blgp:1" : "+a"(acc[j][i]) : "v"(bfr), "v"(afr));
            }
        };
        // ---- even half: B(q+1) has landed; loads younger than it: A(q+1), B(q+2).  The loads of this half overwrite
        // the part that the B fragments of this pair were read from, so every wavefront's reads of it must be over:
        // LDS reads complete in order, and behind the last B read of a pair only TRAIL_READS reads of A follow.
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((nxt ? 8 : 0) + (ISSUE_A.value ? 8 : 0) + EXTRA.value) & lgkmcnt_mask(TRAIL_READS));
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int g = 0; g < 32; ++g) {
            if constexpr (ISSUE_A.value) {
                if ((g & 3) == 0) issue_a(r0, g >> 2);
            }
            if constexpr (nxt) {
                if (g == 2) {
                    if constexpr (par) read_into(fb7_0, b_rd, r2, 7);
                    else read_into(fb7_1, b_rd, r2, 7);
                }
                if (g == 8 + RD_LAG) read_into(fb[0], b_rd, r2, 0);   // behind the MFMAs of block 0
                if (g == 16 + RD_LAG) read_into(fb[1], b_rd, r2, 1);
                if (g == 24 + RD_LAG) read_into(fb[2], b_rd, r2, 2);
            }
            mfma(g);
            if constexpr (ISSUE_A.value) {
                if (g == 30) advance_a();
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- odd half: A(q+1) has landed; loads younger than it: B(q+2), A(q+2).  (Its loads overwrite the part
        // that this pair's A fragments were read from, a whole half ago: no LDS wait.)
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((ISSUE_A.value ? 16 : 0) + EXTRA.value));
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int g = 32; g < 64; ++g) {
            if constexpr (ISSUE_B.value) {
                if ((g & 3) == 0) issue_b(r1, (g - 32) >> 2);
            }
            if constexpr (nxt) {
                if (g == 32 + RD_LAG) read_into(fb[3], b_rd, r2, 3);
                if (g == 40 + RD_LAG) read_into(fb[4], b_rd, r2, 4);
                if (g == 48 + RD_LAG) read_into(fb[5], b_rd, r2, 5);
                if (g == 56 + RD_LAG) read_into(fb[6], b_rd, r2, 6);
                // A blocks at regions 33, 36, 39, 42, 45, 47, 50, 53: between the B reads, all before the last of them
#if defined(DAXQ_F16_SCHED) && DAXQ_F16_SCHED == 1
                constexpr int a_at[8] = {33, 34, 35, 37, 38, 39, 41, 42};
#elif defined(DAXQ_F16_SCHED) && DAXQ_F16_SCHED == 2
                constexpr int a_at[8] = {34, 37, 41, 44, 47, 50, 53, 55};
#else
                constexpr int a_at[8] = {33, 36, 39, 42, 45, 47, 50, 53};
#endif
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (g == a_at[i]) {
                        if constexpr (par) read_into(fa0[i], a_rd, r3, i);
                        else read_into(fa1[i], a_rd, r3, i);
                    }
            }
            mfma(g);
            if constexpr (ISSUE_B.value) {
                if (g == 62) advance_b();
            }
            if (g == 63) {
                const uint32_t o0 = r0, o1 = r1;
                r0 = r2;
                r1 = r3;
                r2 = r4;
                r3 = o0;
                r4 = o1;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- prologue: A(0) and B(0) first, then B(1), A(1), B(2) in ring order; fragments of pair 0 into registers.
    //      (The launcher sends K < 512 to the 32x32x64 kernel: here Q >= 4, every pair of the prologue exists and
    //      pair 0 can be peeled.)
#pragma unroll
    for (int g = 0; g < 8; ++g) issue_a(r1, g);
    advance_a();
#pragma unroll
    for (int g = 0; g < 8; ++g) issue_b(r0, g);
    advance_b();
#pragma unroll
    for (int g = 0; g < 8; ++g) issue_b(r2, g);
    advance_b();
#pragma unroll
    for (int g = 0; g < 8; ++g) issue_a(r3, g);
    advance_a();
#pragma unroll
    for (int g = 0; g < 8; ++g) issue_b(r4, g);
    advance_b();
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(24));
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int j = 0; j < NB - 1; ++j) read_into(fb[j], b_rd, r0, j);
#pragma unroll
    for (int i = 0; i < NB; ++i) read_into(fa0[i], a_rd, r1, i);
    read_into(fb7_0, b_rd, r0, 7);

    // Pair q consumes register set q % 2 and fills the other one.  Pair 0, then the steady pairs 1 .. Q-4 two at a time
    // (odd, even), then one more if their number is odd.  The three pairs of the tail are code paths of their own with
    // fixed sets (even, odd, even): when the steady pairs end on an even one, the fragments it has read for the next
    // pair are moved over to the even set (72 register moves, once per tile).
    pair(No{}, Yes{}, Yes{}, Yes{}, Int<0>{}, Yes{});
    int q = 1;
    for (; q + 4 < Q; q += 2) {
        pair(Yes{}, Yes{}, Yes{}, Yes{}, Int<0>{}, No{});
        pair(No{}, Yes{}, Yes{}, Yes{}, Int<0>{}, No{});
    }
    if (q + 3 < Q) {
        pair(Yes{}, Yes{}, Yes{}, Yes{}, Int<0>{}, No{});
    } else {
#pragma unroll
        for (int i = 0; i < NB; ++i) fa0[i] = fa1[i];
        fb7_0 = fb7_1;
    }
    pair(No{}, Yes{}, No{}, Yes{}, Int<0>{}, No{});  // pair Q-3 (even): the last A loads

    // the epilogue's scales and bias, requested behind the last tile loads (always three loads; a missing bias reads
    // a scale instead and is replaced by -0.0: x + (-0.0) == x bit for bit)
    const float pre_sx = p.sx[m0 + t], pre_sw = p.sw[n0 + t];
    const uint16_t pre_b = (p.bias ? p.bias : reinterpret_cast<const uint16_t*>(p.sw))[n0 + t];
    __builtin_amdgcn_sched_barrier(0);

    pair(Yes{}, No{}, No{}, Yes{}, Int<3>{}, No{});  // pair Q-2 (odd)
    pair(No{}, No{}, No{}, No{}, Int<3>{}, No{});                // pair Q-1 (even)

    // The MFMAs are inline asm, so the compiler cannot count the wait states between one of them and a VALU read of
    // its result: idle cycles first, then every accumulator is passed through an empty statement, which no read of
    // it can move above.
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 7");
#pragma unroll
    for (int j = 0; j < NB; j += 2) {
        asm volatile(""
                     : "+a"(acc[j][0]), "+a"(acc[j][1]), "+a"(acc[j][2]), "+a"(acc[j][3]), "+a"(acc[j][4]), "+a"(acc[j][5]),
                       "+a"(acc[j][6]), "+a"(acc[j][7]), "+a"(acc[j + 1][0]), "+a"(acc[j + 1][1]), "+a"(acc[j + 1][2]),
                       "+a"(acc[j + 1][3]), "+a"(acc[j + 1][4]), "+a"(acc[j + 1][5]), "+a"(acc[j + 1][6]), "+a"(acc[j + 1][7]));
    }
    tile256_epilogue16<DUMP, NB, true>(p, acc, smem, m0, n0, t, wm, wn, lr, kg, pre_sx, pre_sw,
                                       p.bias ? bf16_bits_to_f32(pre_b) : -0.0f);
}

template <bool DUMP, int F8>
static int prepare_tile256f16() {
    static std::atomic<uint64_t> lds_set{0};  // per instantiation
    return ensure_dynamic_lds(reinterpret_cast<const void*>(gemm_tile256f16_kernel<DUMP, F8>), f16::SMEM, lds_set);
}

template <bool DUMP, int F8>
static int launch_tile256f16_impl(const GemmArgs& a, hipStream_t st) {
    auto kern = gemm_tile256f16_kernel<DUMP, F8>;
    if (int rc = prepare_tile256f16<DUMP, F8>()) return rc;
    const int64_t nt = a.grid > 0 ? a.grid : grid_of_order(a);
    if (nt > 0x7fffffff) return fail(DAXQ_ERR_ARG, "gemm: too many tiles");
    hipLaunchKernelGGL(kern, dim3((unsigned)nt), dim3(f16::T), f16::SMEM, st, a);
    return check_launch("gemm_tile256f16");
}

template <int F8>
static int launch_tile256f16(const GemmArgs& a, hipStream_t st) {
    return a.acc ? launch_tile256f16_impl<true, F8>(a, st) : launch_tile256f16_impl<false, F8>(a, st);
}

template <bool FP8, bool DUMP, int F8, bool N16 = false, int BT = 256, bool SPLITK = false, int D = 2, int OUTK = DAXQ_BF16>
static int prepare_tile256s5() {
    static std::atomic<uint64_t> lds_set{0};  // per instantiation
    return ensure_dynamic_lds(reinterpret_cast<const void*>(gemm_tile256s5_kernel<FP8, DUMP, F8, N16, BT, SPLITK, D, OUTK>),
                              (2 * D + 1) * 2 * BT * t5::BKS, lds_set);
}

// split-K launch on 128 tiles: a.splits ranges of K, a.counters zero, a.partials large enough (checked by the caller)
template <bool FP8, int F8>
static int launch_splitk_impl(const GemmArgs& a, hipStream_t st) {
    using namespace t5;
    constexpr int SMEM = NST * 2 * 128 * BKS;
    auto kern = gemm_tile256s5_kernel<FP8, false, F8, !FP8, 128, true>;
    if (int rc = prepare_tile256s5<FP8, false, F8, !FP8, 128, true>()) return rc;
    const int64_t nt = (int64_t)a.tiles_m * a.tiles_n * a.splits;
    if (nt > 0x7fffffff) return fail(DAXQ_ERR_ARG, "gemm: too many workgroups");
    hipLaunchKernelGGL(kern, dim3((unsigned)nt), dim3(T), SMEM, st, a);
    return check_launch("gemm_tile128_splitk");
}

template <bool FP8>
int launch_tile128_splitk(const GemmArgs& a0, int f8, hipStream_t st) {
    GemmArgs a = a0;
    a.tiles_m = (a.m + 127) / 128;
    a.tiles_n = (a.n + 127) / 128;
    if constexpr (FP8) {
        switch (f8) {
            case 1: return launch_splitk_impl<true, 1>(a, st);
            case 2: return launch_splitk_impl<true, 2>(a, st);
            case 3: return launch_splitk_impl<true, 3>(a, st);
            default: return launch_splitk_impl<true, 0>(a, st);
        }
    } else {
        return launch_splitk_impl<false, 0>(a, st);
    }
}

template int launch_tile128_splitk<false>(const GemmArgs&, int, hipStream_t);
template int launch_tile128_splitk<true>(const GemmArgs&, int, hipStream_t);

template <bool FP8, bool DUMP, int F8, bool N16 = false, int BT = 256, int D = 2, int OUTK = DAXQ_BF16>
static int launch_tile256s5_impl(const GemmArgs& a, hipStream_t st) {
    using namespace t5;
    constexpr int SMEM = (2 * D + 1) * 2 * BT * BKS;  // 160 KB (256 tile), 80 KB (128 tile), 144 KB (128 tile, nine stages)
    if (a.out_kind != OUTK) return fail(DAXQ_ERR_ARG, "gemm: this kernel writes output type %d, not %d", OUTK, a.out_kind);
    auto kern = gemm_tile256s5_kernel<FP8, DUMP, F8, N16, BT, false, D, OUTK>;
    if (int rc = prepare_tile256s5<FP8, DUMP, F8, N16, BT, false, D, OUTK>()) return rc;
    const int64_t nt = a.grid > 0 ? a.grid : grid_of_order(a);
    if (nt > 0x7fffffff) return fail(DAXQ_ERR_ARG, "gemm: too many tiles");
    hipLaunchKernelGGL(kern, dim3((unsigned)nt), dim3(T), SMEM, st, a);
    return check_launch("gemm_tile256s5");
}

// 128x128 tiles.  A launch that gives no CU a second workgroup (at most 256 tiles) has the whole LDS of a CU to itself
// and takes the form with nine 16 KB stages (four pairs of slices in flight instead of two) when K is long: measured
// against the five-stage form, M = 512 x N = 5120: K = 5120 22.5 against 23.2 us with the weights near, 31.8 against
// 33.9 us with weights no launch has touched before; K = 13824 71 against 79 us; K = 20480 66 against 76 us; at
// K = 1536 the longer fill and tail cost 4 %, so K < 4096 keeps five stages.  With more tiles two workgroups share a
// CU and its LDS.  A slice takes about 480 cycles here, FP8 (4 MFMAs a slice) and INT8 (16, 256 cycles) alike, and
// what it spends the rest on is its four loads per wavefront, whichever way they go: variants that load into registers
// instead of LDS, read no fragments, wait for no load, drop the barriers or leave the loads to four more wavefronts
// take as long or longer, one without loads 17 against 22 us.
template <bool FP8, int F8, bool N16>
static int launch_tile128(const GemmArgs& a, hipStream_t st) {
    if constexpr (N16) {  // fp16 / fp32 modules (these forms have no accumulator dump: the dispatcher sends that to the generic kernel)
        const bool deep = (a.grid > 0 ? (int64_t)a.grid : (int64_t)a.tiles_m * a.tiles_n) <= 256 && a.k >= 4096;
        if (a.out_kind == DAXQ_F16)
            return deep ? launch_tile256s5_impl<false, false, 0, true, 128, 4, DAXQ_F16>(a, st) : launch_tile256s5_impl<false, false, 0, true, 128, 2, DAXQ_F16>(a, st);
        if (a.out_kind == DAXQ_F32)
            return deep ? launch_tile256s5_impl<false, false, 0, true, 128, 4, DAXQ_F32>(a, st) : launch_tile256s5_impl<false, false, 0, true, 128, 2, DAXQ_F32>(a, st);
    }
    if ((a.grid > 0 ? (int64_t)a.grid : (int64_t)a.tiles_m * a.tiles_n) <= 256 && a.k >= 4096)
        return a.acc ? launch_tile256s5_impl<FP8, true, F8, N16, 128, 4>(a, st) : launch_tile256s5_impl<FP8, false, F8, N16, 128, 4>(a, st);
    return a.acc ? launch_tile256s5_impl<FP8, true, F8, N16, 128>(a, st) : launch_tile256s5_impl<FP8, false, F8, N16, 128>(a, st);
}

// wide:  32x32 MFMAs (INT8 32x32x32, FP8 32x32x64) instead of the 16x16 forms (256 tile only; kept for the tests and for comparisons)
// small: 128x128 tiles (needs m, n >= 128)
// f8:    FP8 operand formats (kF8XE5 | kF8WE5)
template <bool FP8, int F8>
static int launch_tile256s5_f8(const GemmArgs& a, bool wide, bool small, hipStream_t st) {
    if (!small && !wide && a.k >= 512) return launch_tile256f16<F8>(a, st);  // 16x16x128 MFMAs (at least four pairs of slices); wide: the 32x32x64 form
    if (small) return launch_tile128<true, F8, false>(a, st);
    return a.acc ? launch_tile256s5_impl<true, true, F8>(a, st) : launch_tile256s5_impl<true, false, F8>(a, st);
}

template <bool FP8>
static int launch_tile256s5_one(const GemmArgs& a, int f8, bool wide, bool small, hipStream_t st) {
    if constexpr (FP8) {
        switch (f8) {
            case 1: return launch_tile256s5_f8<true, 1>(a, wide, small, st);
            case 2: return launch_tile256s5_f8<true, 2>(a, wide, small, st);
            case 3: return launch_tile256s5_f8<true, 3>(a, wide, small, st);
            default: return launch_tile256s5_f8<true, 0>(a, wide, small, st);
        }
    } else {
        if (small) return launch_tile128<false, 0, true>(a, st);
        if (wide) return a.acc ? launch_tile256s5_impl<false, true, 0>(a, st) : launch_tile256s5_impl<false, false, 0>(a, st);
        if (a.out_kind == DAXQ_F16) return launch_tile256s5_impl<false, false, 0, true, 256, 2, DAXQ_F16>(a, st);
        if (a.out_kind == DAXQ_F32) return launch_tile256s5_impl<false, false, 0, true, 256, 2, DAXQ_F32>(a, st);
        return a.acc ? launch_tile256s5_impl<false, true, 0, true>(a, st) : launch_tile256s5_impl<false, false, 0, true>(a, st);
    }
}

// CUs of the current device (0 if the query fails), asked once per device
static int cu_count() {
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

// Tiles of the last, partial round of a 256x256 launch that go to a second launch on 128x128 tiles; 0 = none.
// One workgroup of 256x256 tiles fills a CU, so a launch of R whole rounds and L more tiles takes R + 1 tile times
// however small L is.  As 4 L quadrants with a CU each (L <= a quarter of the CUs) the L tiles take half a tile time
// or less.  Measured against the single launch (INT8 / e4m3, K = 5120 unless noted):
//   4725 x 13824 (4 rounds + 2 tiles) +5.6 / +6.1 %; 8500 x 4096, K = 2048 (2 + 32) +9.9 / +9.9 %;
//   4095 x 4608, K = 1536 (1 + 32) +10.7 / +9.8 %, K = 8960 +24 / +26 %;
//   20000 x 5120 (6 + 44) +3.3 / +2.4 %; 75600 x 5120 in row groups (23 + 32) -0.6 / -0.8 %: over many rounds the CUs
//   drift apart and the early ones pick the last tiles up, so the cut is taken up to kTailMaxRounds whole rounds;
//   with two quadrants per CU (L up to half the CUs: 4725 x 5120, 1 + 124) -5.3 / -5.9 %: a round of 128x128 tiles
//   at two per CU takes as long as a round of 256x256 tiles, so those launches stay whole.
constexpr int kTailMaxRounds = 8;
static int tail_tiles(const GemmArgs& a, int tail) {
    if (tail == 1 || a.order != 0) return 0;  // the patch orders deal whole patches: their ids are not tile counts
    const int cus = cu_count();
    if (cus < 8) return 0;
    const int64_t tiles = (int64_t)a.tiles_m * a.tiles_n, rounds = tiles / cus, left = tiles - rounds * cus;
    if (rounds < 1 || left == 0 || 4 * left > cus) return 0;
    return (tail == 2 || rounds <= kTailMaxRounds) ? (int)left : 0;
}

// tail: 0 = cut the last partial round off by shape (tail_tiles), 1 = never, 2 = whenever every quadrant gets a CU
template <bool FP8>
int launch_tile256s5(const GemmArgs& a0, int f8, bool wide, bool small, int tail, hipStream_t st) {
    GemmArgs a = a0;
    const int bt = small ? 128 : 256;
    a.tiles_m = (a.m + bt - 1) / bt;
    a.tiles_n = (a.n + bt - 1) / bt;
    a.grid = a.quad_base = 0;
    const int left = small || wide ? 0 : tail_tiles(a, tail);
    if (left == 0) return launch_tile256s5_one<FP8>(a, f8, wide, small, st);
    const int whole = a.tiles_m * a.tiles_n - left;
    a.grid = whole;
    if (int rc = launch_tile256s5_one<FP8>(a, f8, false, false, st)) return rc;
    a.grid = 4 * left;
    a.quad_base = whole + 1;
    return launch_tile256s5_one<FP8>(a, f8, false, true, st);
}

template int launch_tile256s5<false>(const GemmArgs&, int, bool, bool, int, hipStream_t);
template int launch_tile256s5<true>(const GemmArgs&, int, bool, bool, int, hipStream_t);

// Every instantiation the launchers above can pick, prepared on the current device: afterwards no launch changes a
// kernel attribute any more, so the first launch may already sit inside a stream capture.
int prepare_tile256_kernels() {
    int rc = 0;
#define DAXQ_PREP(...) if (!rc) rc = __VA_ARGS__()
    DAXQ_PREP(prepare_tile256<false, false>);
    DAXQ_PREP(prepare_tile256<false, true>);
    DAXQ_PREP(prepare_tile256<true, false>);
    DAXQ_PREP(prepare_tile256<true, true>);
    DAXQ_PREP(prepare_tile256<true, false, true>);
    DAXQ_PREP(prepare_tile256<true, true, true>);
    DAXQ_PREP(prepare_tile256s5<false, false, 0, true, 256>);
    DAXQ_PREP(prepare_tile256s5<false, true, 0, true, 256>);
    DAXQ_PREP(prepare_tile256s5<false, false, 0, false, 256>);
    DAXQ_PREP(prepare_tile256s5<false, true, 0, false, 256>);
    DAXQ_PREP(prepare_tile256s5<false, false, 0, true, 128>);
    DAXQ_PREP(prepare_tile256s5<false, true, 0, true, 128>);
    DAXQ_PREP(prepare_tile256s5<false, false, 0, true, 128, false, 4>);
    DAXQ_PREP(prepare_tile256s5<false, true, 0, true, 128, false, 4>);
    DAXQ_PREP(prepare_tile256s5<false, false, 0, true, 256, false, 2, DAXQ_F16>);
    DAXQ_PREP(prepare_tile256s5<false, false, 0, true, 128, false, 2, DAXQ_F16>);
    DAXQ_PREP(prepare_tile256s5<false, false, 0, true, 128, false, 4, DAXQ_F16>);
    DAXQ_PREP(prepare_tile256s5<false, false, 0, true, 256, false, 2, DAXQ_F32>);
    DAXQ_PREP(prepare_tile256s5<false, false, 0, true, 128, false, 2, DAXQ_F32>);
    DAXQ_PREP(prepare_tile256s5<false, false, 0, true, 128, false, 4, DAXQ_F32>);
    DAXQ_PREP(prepare_tile256s5<false, false, 0, true, 128, true>);
#define DAXQ_PREP_F8(F8)                                         \
    DAXQ_PREP(prepare_tile256s5<true, false, F8, false, 128, true>); \
    DAXQ_PREP(prepare_tile256s5<true, false, F8, false, 256>);   \
    DAXQ_PREP(prepare_tile256s5<true, true, F8, false, 256>);    \
    DAXQ_PREP(prepare_tile256s5<true, false, F8, false, 128>);   \
    DAXQ_PREP(prepare_tile256s5<true, true, F8, false, 128>);    \
    DAXQ_PREP(prepare_tile256s5<true, false, F8, false, 128, false, 4>); \
    DAXQ_PREP(prepare_tile256s5<true, true, F8, false, 128, false, 4>)
#define DAXQ_PREP_F16(F8)                      \
    DAXQ_PREP(prepare_tile256f16<false, F8>); \
    DAXQ_PREP(prepare_tile256f16<true, F8>)
    DAXQ_PREP_F16(0);
    DAXQ_PREP_F16(1);
    DAXQ_PREP_F16(2);
    DAXQ_PREP_F16(3);
#undef DAXQ_PREP_F16
    DAXQ_PREP_F8(0);
    DAXQ_PREP_F8(1);
    DAXQ_PREP_F8(2);
    DAXQ_PREP_F8(3);
#undef DAXQ_PREP_F8
#undef DAXQ_PREP
    return rc;
}

// the kernel applies: both dimensions hold a whole tile and the 32-bit row offsets cannot overflow
bool tile256_applies(const GemmArgs& a) {
    return a.m >= t256::BM && a.n >= t256::BN && a.lda < (1 << 26) && a.ldb < (1 << 26);
}

template int launch_tile256<false>(const GemmArgs&, bool, hipStream_t);
template int launch_tile256<true>(const GemmArgs&, bool, hipStream_t);

}  // namespace daxq
