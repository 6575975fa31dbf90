// Tiled INT8 W8A8 GEMM for gfx950: the kernel the large DiT shapes run on (256x256 tiles), the same pipeline on
// 128x128 tiles for launches with too few of those to fill the CUs, and its split-K form (INT8 and FP8).
// FP8 launches without split-K run gemm_tile_fp8.hip.
//
// Work decomposition
//   workgroup  BT x BT outputs (BT = 256 or 128), 4 wavefronts (one per SIMD) in a 2 x 2 grid
//   wavefront  BT/2 x BT/2 outputs: INT8 as blocks of 16x16 (v_mfma_i32_16x16x64_i8, 8 x 8 of them for BT = 256: 256
//              accumulator registers), the FP8 split-K form as blocks of 32x32 (v_mfma_f32_32x32x64_f8f6f4)
// A 2 x 2 wave grid is what minimises LDS reads per MFMA for a square tile.
//
// Which tile a workgroup computes is a launch argument (GemmArgs::order, gemm_tile.h): groups of tile rows per XCD, or
// the banded order of tile_order.h that gives the 32 CUs of an XCD a patch of 32 tiles, the eight XCDs on the same
// activation rows and on different weight columns; the large launches take the banded one.
//
// Tiles at the M / N edge are shifted inwards (origin min(tile*BT, dim-BT)) instead of being predicated: the overlap
// rows are computed twice with identical results.  Shapes with M < 128 or N < 128 take the generic kernel in
// gemm_w8a8.hip.
#include "gemm_tile.h"
#include "gemm_tile256x128.h"

namespace daxq {

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

// ---------------------------------------------------------------------------------------------
// K in 64-byte slices through five 32 KB LDS stages (all 160 KB): the LDS holds the slice being read plus four more,
// and the load stream is even: 8 loads per 64-byte slice, one every eighth MFMA (INT8).
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
__device__ __forceinline__ void gemm_tile256s5_body(const GemmArgs& p, const int block) {
    static_assert(OUTK == DAXQ_BF16 || (N16 && !SPLITK && !DUMP), "fp16 / fp32 outputs exist in the 16x16 int8 form");
    using namespace t5;
    static_assert(!(FP8 && N16), "the 16x16 form exists for INT8 only");
    static_assert(FP8 ? SPLITK : N16, "INT8 runs the 16x16 form; FP8 comes here for split-K only");
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
    int tile_id = block, split = 0, klen = p.k;  // klen: bytes of K this workgroup covers, a multiple of 128
    int m0, n0;
    if constexpr (SPLITK) {
        static_assert(BT == 128 && !DUMP, "split-K exists on 128 tiles, without the accumulator dump");
        tile_id = block / p.splits;
        split = block - tile_id * p.splits;
        klen = p.k / p.splits;
        int tm, tn;
        tile_of_block(p.gm, tile_id, p.tiles_m, p.tiles_n, tm, tn);
        m0 = tm * BT, n0 = tn * BT;
        m0 = m0 + BT <= p.m ? m0 : p.m - BT;
        n0 = n0 + BT <= p.n ? n0 : p.n - BT;
    } else {
        if (!tile_origin<BT>(p, tile_id, m0, n0)) return;  // padding slot (before any barrier)
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
                // B block j, A block i: consecutive MFMAs share the weight fragment (holding the activation fragment instead
                // measured the same: 2985 - 2994 against 2997 - 3000 T-op/s)
                const int j = g / NB, i = g % NB;
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
        uint64_t* mine = static_cast<uint64_t*>(p.partials) + ((int64_t)block * NV * 256 + t) * 2;
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
        tile_epilogue16<DUMP, NB, NB, false, OUTK>(p, acc, smem, m0, n0, t, wm, wn, lr, lane >> 4, pre_sx, pre_sw,
                                                  !p.bias ? -0.0f : OUTK == DAXQ_F32 ? __uint_as_float(pre_b) : OUTK == DAXQ_F16 ? f16_bits_to_f32((uint16_t)pre_b) : bf16_bits_to_f32(pre_b));
    else
        tile256_epilogue<FP8, DUMP, NB>(p, acc, smem, m0, n0, t, wm, wn, l31, hi, pre_sx, pre_sw,
                                        p.bias ? bf16_bits_to_f32(pre_b) : -0.0f);
}

template <bool FP8, bool DUMP, int F8, bool N16 = false, int BT = 256, bool SPLITK = false, int D = 2, int OUTK = DAXQ_BF16>
__global__ __launch_bounds__(256) void gemm_tile256s5_kernel(const GemmArgs p) {
    gemm_tile256s5_body<FP8, DUMP, F8, N16, BT, SPLITK, D, OUTK>(p, (int)blockIdx.x);
}

// One grid for a launch of few rounds whose left-over tiles run as halves (tail_half_tiles): workgroups 0 .. p.grid - 1
// compute whole 256x256 tiles, the rest the 256x128 halves of the tiles from id quad_base - 1 on.  The halves start on
// the CUs that finish their whole tiles first instead of behind the whole first kernel.
template <bool DUMP, int OUTK>
__global__ __launch_bounds__(256) void gemm_tile256_then_halves_kernel(const GemmArgs p) {
    if ((int)blockIdx.x < p.grid) gemm_tile256s5_body<false, DUMP, 0, true, 256, false, 2, OUTK>(p, (int)blockIdx.x);
    else gemm_tile256x128_body<DUMP, OUTK>(p, (int)blockIdx.x - p.grid);
}

// The same for left-over tiles that run as 128x128 quadrants (tail_tiles): workgroups 0 .. p.grid - 1 compute whole
// tiles, the rest the quadrants of the tiles from id quad_base - 1 on (D: pairs of slices the quadrants keep in flight).
template <bool DUMP, int OUTK, int D>
__global__ __launch_bounds__(256) void gemm_tile256_then_quadrants_kernel(const GemmArgs p) {
    if ((int)blockIdx.x < p.grid) gemm_tile256s5_body<false, DUMP, 0, true, 256, false, 2, OUTK>(p, (int)blockIdx.x);
    else gemm_tile256s5_body<false, DUMP, 0, true, 128, false, D, OUTK>(p, (int)blockIdx.x - p.grid);
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
    const int64_t nt = grid_of_order(a);
    if (nt > 0x7fffffff) return fail(DAXQ_ERR_ARG, "gemm: too many tiles");
    hipLaunchKernelGGL(kern, dim3((unsigned)nt), dim3(T), SMEM, st, a);
    return check_launch("gemm_tile256s5");
}

// 128x128 tiles.  A launch that gives no CU a second workgroup (at most 256 tiles) has the whole LDS of a CU to itself
// and takes the form with nine 16 KB stages (four pairs of slices in flight instead of two) when K is long: measured
// against the five-stage form, M = 512 x N = 5120: K = 5120 22.5 against 23.2 us with the weights near, 31.8 against
// 33.9 us with weights no launch has touched before; K = 13824 71 against 79 us; K = 20480 66 against 76 us; at
// K = 1536 the longer fill and tail cost 4 %, so K < 4096 keeps five stages.  With more tiles two workgroups share a
// CU and its LDS.  A slice takes about 480 cycles here (16 MFMAs: 256 cycles), and what it spends the rest on is its
// four loads per wavefront, whichever way they go: variants that load into registers instead of LDS, read no
// fragments, wait for no load, drop the barriers or leave the loads to four more wavefronts take as long or longer,
// one without loads 17 against 22 us.
template <int OUTK>
static int launch_i8_128_out(const GemmArgs& a, hipStream_t st) {
    const bool deep = (int64_t)a.tiles_m * a.tiles_n <= 256 && a.k >= 4096;
    if constexpr (OUTK == DAXQ_BF16) {
        if (a.acc) return deep ? launch_tile256s5_impl<false, true, 0, true, 128, 4>(a, st) : launch_tile256s5_impl<false, true, 0, true, 128, 2>(a, st);
    }
    return deep ? launch_tile256s5_impl<false, false, 0, true, 128, 4, OUTK>(a, st) : launch_tile256s5_impl<false, false, 0, true, 128, 2, OUTK>(a, st);
}

// small: 128x128 tiles (needs m, n >= 128)
static int launch_i8_one(const GemmArgs& a, bool small, hipStream_t st) {
    if (a.acc && a.out_kind != DAXQ_BF16) return fail(DAXQ_ERR_ARG, "gemm: the accumulator dump exists with bf16 outputs");
    if (small) {
        if (a.out_kind == DAXQ_F16) return launch_i8_128_out<DAXQ_F16>(a, st);
        if (a.out_kind == DAXQ_F32) return launch_i8_128_out<DAXQ_F32>(a, st);
        return launch_i8_128_out<DAXQ_BF16>(a, st);
    }
    if (a.out_kind == DAXQ_F16) return launch_tile256s5_impl<false, false, 0, true, 256, 2, DAXQ_F16>(a, st);
    if (a.out_kind == DAXQ_F32) return launch_tile256s5_impl<false, false, 0, true, 256, 2, DAXQ_F32>(a, st);
    return a.acc ? launch_tile256s5_impl<false, true, 0, true>(a, st) : launch_tile256s5_impl<false, false, 0, true>(a, st);
}

// The last, partial round of a launch of 256x256 tiles in smaller pieces with a CU each: tail_tiles (quadrants) and
// tail_half_tiles (halves) in gemm_tile.h say which tiles, the kernels above run them in the same grid, behind the
// whole tiles.  tail: 0 = by shape, 1 = never, 2 = whenever every piece gets a CU
template <bool DUMP, int OUTK>
static int prepare_then_halves() {
    static std::atomic<uint64_t> lds_set{0};  // per instantiation
    return ensure_dynamic_lds(reinterpret_cast<const void*>(gemm_tile256_then_halves_kernel<DUMP, OUTK>), 5 * 2 * 256 * t5::BKS, lds_set);
}

template <bool DUMP, int OUTK>
static int launch_then_halves_impl(const GemmArgs& a, int64_t nt, hipStream_t st) {
    if (int rc = prepare_then_halves<DUMP, OUTK>()) return rc;
    hipLaunchKernelGGL((gemm_tile256_then_halves_kernel<DUMP, OUTK>), dim3((unsigned)nt), dim3(t5::T), 5 * 2 * 256 * t5::BKS, st, a);
    return check_launch("gemm_tile256_then_halves");
}

// `whole` 256x256 tiles of the row-group order, then the two halves of each of the `halves` tiles behind them, in one grid
static int launch_then_halves(const GemmArgs& a0, int whole, int halves, hipStream_t st) {
    GemmArgs a = a0;
    a.grid = whole;
    a.quad_base = whole + 1;
    const int64_t nt = (int64_t)whole + 2 * (int64_t)halves;
    if (nt > 0x7fffffff) return fail(DAXQ_ERR_ARG, "gemm: too many tiles");
    if (a.acc && a.out_kind != DAXQ_BF16) return fail(DAXQ_ERR_ARG, "gemm: the accumulator dump exists with bf16 outputs");
    if (a.out_kind == DAXQ_F16) return launch_then_halves_impl<false, DAXQ_F16>(a, nt, st);
    if (a.out_kind == DAXQ_F32) return launch_then_halves_impl<false, DAXQ_F32>(a, nt, st);
    return a.acc ? launch_then_halves_impl<true, DAXQ_BF16>(a, nt, st) : launch_then_halves_impl<false, DAXQ_BF16>(a, nt, st);
}

template <bool DUMP, int OUTK, int D>
static int prepare_then_quadrants() {
    static std::atomic<uint64_t> lds_set{0};  // per instantiation
    return ensure_dynamic_lds(reinterpret_cast<const void*>(gemm_tile256_then_quadrants_kernel<DUMP, OUTK, D>), 5 * 2 * 256 * t5::BKS, lds_set);
}

template <bool DUMP, int OUTK, int D>
static int launch_then_quadrants_impl(const GemmArgs& a, int64_t nt, hipStream_t st) {
    if (int rc = prepare_then_quadrants<DUMP, OUTK, D>()) return rc;
    hipLaunchKernelGGL((gemm_tile256_then_quadrants_kernel<DUMP, OUTK, D>), dim3((unsigned)nt), dim3(t5::T), 5 * 2 * 256 * t5::BKS, st, a);
    return check_launch("gemm_tile256_then_quadrants");
}

template <int D>
static int launch_then_quadrants_out(const GemmArgs& a, int64_t nt, hipStream_t st) {
    if (a.acc && a.out_kind != DAXQ_BF16) return fail(DAXQ_ERR_ARG, "gemm: the accumulator dump exists with bf16 outputs");
    if (a.out_kind == DAXQ_F16) return launch_then_quadrants_impl<false, DAXQ_F16, D>(a, nt, st);
    if (a.out_kind == DAXQ_F32) return launch_then_quadrants_impl<false, DAXQ_F32, D>(a, nt, st);
    return a.acc ? launch_then_quadrants_impl<true, DAXQ_BF16, D>(a, nt, st) : launch_then_quadrants_impl<false, DAXQ_BF16, D>(a, nt, st);
}

// `whole` 256x256 tiles of the row-group order, then the four quadrants of each of the `left` tiles behind them, in one
// grid; the quadrants have a CU each and take the deep ring when K is long (launch_i8_128_out)
static int launch_then_quadrants(const GemmArgs& a0, int whole, int left, hipStream_t st) {
    GemmArgs a = a0;
    a.grid = whole;
    a.quad_base = whole + 1;
    const int64_t nt = (int64_t)whole + 4 * (int64_t)left;
    if (nt > 0x7fffffff) return fail(DAXQ_ERR_ARG, "gemm: too many tiles");
    return a.k >= 4096 ? launch_then_quadrants_out<4>(a, nt, st) : launch_then_quadrants_out<2>(a, nt, st);
}

// Every 256x256 tile as its two 256x128 halves (needs m, n >= 256): the grid of launch_then_halves without whole tiles
int launch_halves_i8(const GemmArgs& a0, hipStream_t st) {
    GemmArgs a = a0;
    a.tiles_m = (a.m + 255) / 256;
    a.tiles_n = (a.n + 255) / 256;
    a.order = kOrderRowGroups;
    const int64_t tiles = (int64_t)a.tiles_m * a.tiles_n;
    if (tiles > 0x3fffffff) return fail(DAXQ_ERR_ARG, "gemm: too many tiles");
    return launch_then_halves(a, 0, (int)tiles, st);
}

int launch_tile_i8(const GemmArgs& a0, bool small, int tail, hipStream_t st) {
    GemmArgs a = a0;
    const int bt = small ? 128 : 256;
    a.tiles_m = (a.m + bt - 1) / bt;
    a.tiles_n = (a.n + bt - 1) / bt;
    a.grid = a.quad_base = 0;
    if (small) a.order = kOrderRowGroups;
    const int left = small ? 0 : tail_tiles(a, tail);
    if (left == 0) {
        const int halves = small ? 0 : tail_half_tiles(a, tail);
        if (halves == 0) return launch_i8_one(a, small, st);
        return launch_then_halves(a, a.tiles_m * a.tiles_n - halves, halves, st);
    }
    return launch_then_quadrants(a, a.tiles_m * a.tiles_n - left, left, st);
}

// Every instantiation the launchers above can pick, prepared on the current device: afterwards no launch changes a
// kernel attribute any more, so the first launch may already sit inside a stream capture.
int prepare_tile256_kernels() {
    int rc = 0;
#define DAXQ_PREP(...) if (!rc) rc = __VA_ARGS__()
    DAXQ_PREP(prepare_tile256s5<false, false, 0, true, 256>);
    DAXQ_PREP(prepare_tile256s5<false, true, 0, true, 256>);
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
    DAXQ_PREP(prepare_tile256s5<true, false, 0, false, 128, true>);
    DAXQ_PREP(prepare_tile256s5<true, false, 1, false, 128, true>);
    DAXQ_PREP(prepare_tile256s5<true, false, 2, false, 128, true>);
    DAXQ_PREP(prepare_tile256s5<true, false, 3, false, 128, true>);
    DAXQ_PREP(prepare_then_halves<false, DAXQ_BF16>);
    DAXQ_PREP(prepare_then_halves<true, DAXQ_BF16>);
    DAXQ_PREP(prepare_then_halves<false, DAXQ_F16>);
    DAXQ_PREP(prepare_then_halves<false, DAXQ_F32>);
    DAXQ_PREP(prepare_then_quadrants<false, DAXQ_BF16, 2>);
    DAXQ_PREP(prepare_then_quadrants<true, DAXQ_BF16, 2>);
    DAXQ_PREP(prepare_then_quadrants<false, DAXQ_F16, 2>);
    DAXQ_PREP(prepare_then_quadrants<false, DAXQ_F32, 2>);
    DAXQ_PREP(prepare_then_quadrants<false, DAXQ_BF16, 4>);
    DAXQ_PREP(prepare_then_quadrants<true, DAXQ_BF16, 4>);
    DAXQ_PREP(prepare_then_quadrants<false, DAXQ_F16, 4>);
    DAXQ_PREP(prepare_then_quadrants<false, DAXQ_F32, 4>);
#undef DAXQ_PREP
    return rc;
}

// the tiled kernels apply: both dimensions hold a whole 256 tile and the 32-bit row offsets cannot overflow
bool tile256_applies(const GemmArgs& a) {
    return a.m >= 256 && a.n >= 256 && a.lda < (1 << 26) && a.ldb < (1 << 26);
}

}  // namespace daxq
