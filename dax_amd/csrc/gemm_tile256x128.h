// W8A8 GEMM on half tiles of 256 x 128 outputs: the left-over tiles of a launch of few rounds (INT8 first, FP8 below),
// as device functions that the kernels of gemm_tile256.hip and gemm_tile_fp8.hip run in the workgroups behind those of
// the whole tiles.
//
// A launch of 256x256 tiles that leaves L tiles over after its whole rounds of workgroups pays a whole tile time for
// them.  Up to a quarter of the CUs' worth of such tiles run as 128x128 quadrants with a CU each (gemm_tile256.hip);
// between a quarter and a half they run here, as 2 L halves of 256 rows x 128 columns with a CU each: four wavefronts
// in a 2 x 2 grid with 128 x 64 outputs each (128 accumulator registers), K through five 24 KB LDS stages with the load
// stream of the large kernel (12 loads per thread and pair of slices: the 8 of the activation rows during the even
// slice, the 4 of the weight rows during the odd one).  A half tile has 12 fragment reads per 32 MFMAs where the whole
// tile has 16 per 64, so it runs at about 0.7 of the whole tile's pace: 0.7 of a tile time instead of one.
// Same arithmetic as the large kernel: int32 accumulators, identical outputs.
#pragma once

#include "gemm_tile.h"

namespace daxq {

namespace h2 {
constexpr int BKS = 64, BM = 256, BN = 128, T = 256, NSTG = 5;
constexpr int A_BYTES = BM * BKS, B_BYTES = BN * BKS, STAGE = A_BYTES + B_BYTES;  // 16 KB + 8 KB per stage
constexpr int NBI = 8, NBJ = 4;                         // 16-row blocks of a wavefront: activation rows, weight rows
constexpr int NREG = NBI * NBJ;                         // MFMAs = scheduling regions per slice and wavefront
constexpr int A_LOADS = 8, B_LOADS = 4;                 // DMA loads per thread and pair of slices: activation rows, weight rows
constexpr int PAIR_LOADS = A_LOADS + B_LOADS;
constexpr int SMEM = NSTG * STAGE;
}  // namespace h2

template <bool DUMP, int OUTK>
__device__ __forceinline__ void gemm_tile256x128_body(const GemmArgs& p, const int half_id) {
    static_assert(OUTK == DAXQ_BF16 || !DUMP, "the accumulator dump exists with bf16 outputs");
    using namespace h2;
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    // half (half_id & 1) of the 256x256 tile quad_base - 1 + half_id / 2 of the row-group order
    int tm, tn;
    tile_of_block(p.gm, p.quad_base - 1 + (half_id >> 1), p.tiles_m, p.tiles_n, tm, tn);
    int m0 = tm * 256, n0 = tn * 256;
    m0 = m0 + 256 <= p.m ? m0 : p.m - 256;
    n0 = (n0 + 256 <= p.n ? n0 : p.n - 256) + (half_id & 1) * 128;

    // ---- HBM side.  One wave instruction fills 1 KB of LDS = 16 rows x 64 B: lane l -> row l/4, stored chunk l%4,
    //      i.e. global chunk (l%4) ^ ((row>>1)&3).  Instruction j of a thread covers tile rows j*64 + t/4.
    const uint32_t gsw = (uint32_t)(((t & 3) ^ ((t >> 3) & 3)) << 4);
    uint32_t voff_a = (uint32_t)(t >> 2) * (uint32_t)p.lda + gsw;
    uint32_t voff_b = (uint32_t)(t >> 2) * (uint32_t)p.ldb + gsw;
    uint32_t voff_a1 = voff_a + BKS, voff_b1 = voff_b + BKS;  // second half of the 128-byte line
    const uint8_t* abase = p.a + (int64_t)m0 * p.lda;
    const uint8_t* bbase = p.b + (int64_t)n0 * p.ldb;
    const int64_t a_step = 64 * p.lda, b_step = 64 * p.ldb;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(DAXQ_LDS uint8_t*)smem;
    const uint32_t wave_lds = lds0 + (uint32_t)__builtin_amdgcn_readfirstlane(wave * 1024);
    // load g of a pair (12): 0-7 activation rows, 8-11 weight rows; 64-row block (g/2) % 4, half g%2 -> stage o0 / o1
    auto issue_one = [&](uint32_t o0, uint32_t o1, int g) {
        const int opnd = g >= A_LOADS, j = ((opnd ? g - A_LOADS : g) >> 1), half = g & 1;
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

    // ---- LDS side: activation row wm*128 + i*16 + l%16, weight row wn*64 + j*16 + l%16; the lane's K chunk is l/16
    const int lr = lane & 15;
    const int gq = (lr >> 1) & 3;
    const uint8_t* a_rd = smem + (wm * 128 + lr) * BKS + (((lane >> 4) ^ gq) << 4);
    const uint8_t* b_rd = smem + A_BYTES + (wn * 64 + lr) * BKS + (((lane >> 4) ^ gq) << 4);
    // fragment f of a slice: 0-7 activation block f, 8-11 weight block f-8
    auto read_frag = [&](uint32_t o, int f, v4i (&af)[NBI], v4i (&bf)[NBJ]) {
        if (f < NBI) af[f] = *reinterpret_cast<const v4i*>(a_rd + o + f * 16 * BKS);
        else bf[f - NBI] = *reinterpret_cast<const v4i*>(b_rd + o + (f - NBI) * 16 * BKS);
    };

    v4i acc[NBJ][NBI];
    v4i fa0[NBI] = {}, fb0[NBJ] = {}, fa1[NBI] = {}, fb1[NBJ] = {};  // fragment sets by slice parity

    const int S = p.k / BKS;  // slices; even because K is a multiple of 128
    uint32_t st[NSTG];        // stage offsets of slices s .. s+3 and, last, of slice s-1 (s = the even slice of the pair)
#pragma unroll
    for (int i = 0; i < NSTG; ++i) st[i] = i * STAGE;

    // One slice (see gemm_tile256.hip for the scheme).  ODD: slice parity.  ISSUE: start half of pair (s+4, s+5).
    // NEXT: slice s+1 exists.  YOUNG: tile loads issued behind those of slice s+1 that may stay in flight.  EXTRA:
    // younger loads that are not tile loads.  FIRST: slice 0, its MFMAs start from zero.
    auto slice = [&](auto ODD, auto ISSUE, auto NEXT, auto YOUNG, auto EXTRA, auto FIRST, uint32_t o_next, uint32_t o_ld0, uint32_t o_ld1)
                     __attribute__((always_inline)) {
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(YOUNG.value + EXTRA.value) & lgkmcnt0_mask());
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int g = 0; g < NREG; ++g) {
            if constexpr (ISSUE.value) {  // even slice: the 8 activation loads, one every 4 regions; odd: the 4 weight loads, every 8
                if constexpr (ODD.value) {
                    if (g % (NREG / B_LOADS) == 0) issue_one(o_ld0, o_ld1, A_LOADS + g / (NREG / B_LOADS));
                } else {
                    if (g % (NREG / A_LOADS) == 0) issue_one(o_ld0, o_ld1, g / (NREG / A_LOADS));
                }
            }
            if constexpr (NEXT.value) {  // 12 reads, one every second region
                if (g % 2 == 0 && g / 2 < NBI + NBJ) {
                    if constexpr (ODD.value) read_frag(o_next, g / 2, fa0, fb0);
                    else read_frag(o_next, g / 2, fa1, fb1);
                }
            }
            const int j = g / NBI, i = g % NBI;
            const v4i bfr = ODD.value ? fb1[j] : fb0[j];
            const v4i afr = ODD.value ? fa1[i] : fa0[i];
            if constexpr (FIRST.value)
                asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, 0" : "=a"(acc[j][i]) : "v"(bfr), "v"(afr));
            else
                asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(acc[j][i]) : "v"(bfr), "v"(afr));
            if constexpr (ISSUE.value) {
                if (g == NREG - 2) {
                    if constexpr (ODD.value) advance_b();
                    else advance_a();
                }
            }
            if constexpr (ODD.value) {
                if (g == NREG - 1) {
                    const uint32_t r0 = st[0], r1 = st[1];
#pragma unroll
                    for (int i2 = 0; i2 + 2 < NSTG; ++i2) st[i2] = st[i2 + 2];
                    st[NSTG - 2] = r0;
                    st[NSTG - 1] = r1;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto pair = [&](auto ISSUE, auto YOUNG_E, auto YOUNG_O, auto NEXT_O, auto EXTRA, auto FIRST) __attribute__((always_inline)) {
        slice(No{}, ISSUE, Yes{}, YOUNG_E, EXTRA, FIRST, st[1], st[NSTG - 1], st[0]);
        slice(Yes{}, ISSUE, NEXT_O, YOUNG_O, EXTRA, No{}, st[2], st[NSTG - 1], st[0]);
    };
    typedef Int<PAIR_LOADS> SteadyE;  // one whole pair younger than the pair of slice s+1
    typedef Int<A_LOADS> SteadyO;     // the activation half of the newest pair

    // ---- prologue: pairs 0 and 1 in flight, pair 0 landed, fragments of slice 0 in set 0
#pragma unroll
    for (int g = 0; g < PAIR_LOADS; ++g) issue_one(0, STAGE, g);
    advance_a();
    advance_b();
    if (S >= 4) {
#pragma unroll
        for (int g = 0; g < PAIR_LOADS; ++g) issue_one(2 * STAGE, 3 * STAGE, g);
        advance_a();
        advance_b();
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(PAIR_LOADS));
    } else {
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    }
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int f = 0; f < NBI + NBJ; ++f) read_frag(0, f, fa0, fb0);

    const int Q = S >> 1;  // pairs
    if (Q >= 3) {
        pair(Yes{}, SteadyE{}, SteadyO{}, Yes{}, Int<0>{}, Yes{});
    } else {  // short K: no pair to peel, clear the accumulators instead
#pragma unroll
        for (int j = 0; j < NBJ; ++j)
#pragma unroll
            for (int i = 0; i < NBI; ++i) acc[j][i] = v4i{};
    }
    for (int q = 1; q + 2 < Q; ++q) pair(Yes{}, SteadyE{}, SteadyO{}, Yes{}, Int<0>{}, No{});

    // the epilogue's scales and bias, requested behind the last tile loads (always three loads per thread: a missing
    // bias reads a scale instead and is replaced by -0.0)
    const int tn2 = t & (BN - 1);  // (the upper half of the threads repeats the lower half's weight-side loads: the counts of the waits hold)
    const float pre_sx = p.sx[m0 + t], pre_sw = p.sw[n0 + tn2];
    uint32_t pre_b;  // the bias element's bits: bf16 / fp16, or fp32
    if constexpr (OUTK == DAXQ_F32) pre_b = __float_as_uint((p.bias ? reinterpret_cast<const float*>(p.bias) : p.sw)[n0 + tn2]);
    else pre_b = (p.bias ? p.bias : reinterpret_cast<const uint16_t*>(p.sw))[n0 + tn2];
    __builtin_amdgcn_sched_barrier(0);

    if (Q >= 2) pair(No{}, Int<PAIR_LOADS>{}, Int<0>{}, Yes{}, Int<3>{}, No{});
    pair(No{}, Int<0>{}, Int<0>{}, No{}, Int<3>{}, No{});

    // the MFMAs are inline asm: nothing tells the compiler how long their results take (see gemm_tile256.hip)
    asm volatile("s_nop 15\n\ts_nop 7");
#pragma unroll
    for (int j = 0; j < NBJ; ++j)
        asm volatile(""
                     : "+a"(acc[j][0]), "+a"(acc[j][1]), "+a"(acc[j][2]), "+a"(acc[j][3]), "+a"(acc[j][4]), "+a"(acc[j][5]),
                       "+a"(acc[j][6]), "+a"(acc[j][7]));
    tile_epilogue16<DUMP, NBJ, NBI, false, OUTK>(p, acc, smem, m0, n0, t, wm, wn, lr, lane >> 4, pre_sx, pre_sw,
                                                 !p.bias ? -0.0f : OUTK == DAXQ_F32 ? __uint_as_float(pre_b) : OUTK == DAXQ_F16 ? f16_bits_to_f32((uint16_t)pre_b) : bf16_bits_to_f32(pre_b));
}

// ---------------------------------------------------------------------------------------------------------------------
// The same half tile for FP8 operands (v_mfma_f32_16x16x128_f8f6f4).  An output element is the same sequence of MFMAs
// over the same K bytes in the same register positions as in gemm_tile_fp8.hip -- one MFMA per pair of 64-byte slices,
// a lane's fragments holding chunk l/16 of the pair's first slice, then of its second -- so its bits do not depend on
// which of the kernels computed it.  With 128 accumulator registers both operands' fragments fit twice (12 x 8 x 2):
// the fragments of pair q+1 are read during the MFMAs of pair q, the LDS holds three pairs (48 KB each: pair q+1
// landed, q+2 in flight, and the slot of pair q, which was read a pair ago, taking the loads of q+3), one barrier per pair.
namespace h2f {
constexpr int BKS = 64, BM = 256, BN = 128, T = 256;
constexpr int A_HALF = BM * BKS, B_HALF = BN * BKS;          // one slice of an operand: 16 KB / 8 KB
constexpr int A_PART = 2 * A_HALF, SLOT = A_PART + 2 * B_HALF;  // a pair: 32 KB of activation rows, 16 KB of weight rows
constexpr int NBI = 8, NBJ = 4, NREG = NBI * NBJ;
constexpr int A_LOADS = 8, B_LOADS = 4, PAIR_LOADS = A_LOADS + B_LOADS;
constexpr int SMEM = 3 * SLOT;
}  // namespace h2f

template <bool DUMP, int F8, int OUTK>
__device__ __forceinline__ void gemm_tile256x128_fp8_body(const GemmArgs& p, const int half_id) {
    static_assert(OUTK == DAXQ_BF16 || !DUMP, "the accumulator dump exists with bf16 outputs");
    using namespace h2f;
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    int tm, tn;
    tile_of_block(p.gm, p.quad_base - 1 + (half_id >> 1), p.tiles_m, p.tiles_n, tm, tn);
    int m0 = tm * 256, n0 = tn * 256;
    m0 = m0 + 256 <= p.m ? m0 : p.m - 256;
    n0 = (n0 + 256 <= p.n ? n0 : p.n - 256) + (half_id & 1) * 128;

    const uint32_t gsw = (uint32_t)(((t & 3) ^ ((t >> 3) & 3)) << 4);
    uint32_t voff_a = (uint32_t)(t >> 2) * (uint32_t)p.lda + gsw;
    uint32_t voff_b = (uint32_t)(t >> 2) * (uint32_t)p.ldb + gsw;
    uint32_t voff_a1 = voff_a + BKS, voff_b1 = voff_b + BKS;  // second half of the 128-byte line
    const uint8_t* abase = p.a + (int64_t)m0 * p.lda;
    const uint8_t* bbase = p.b + (int64_t)n0 * p.ldb;
    const int64_t a_step = 64 * p.lda, b_step = 64 * p.ldb;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(DAXQ_LDS uint8_t*)smem;
    const uint32_t wave_lds = lds0 + (uint32_t)__builtin_amdgcn_readfirstlane(wave * 1024);
    // load g of a pair (12): 0-7 activation rows, 8-11 weight rows; 64-row block, then slice g%2 of the pair (the two
    // halves of a 128-byte line by consecutive instructions).  Address = uniform row-block base (SGPR pair) + per-lane
    // 32-bit offset: no VALU work per load.
    auto issue_one = [&](uint32_t slot, int g) {
        const int opnd = g >= A_LOADS, gg = opnd ? g - A_LOADS : g, j = gg >> 1, half = gg & 1;
        const uint8_t* src = opnd ? bbase + j * b_step : abase + j * a_step;
        const uint32_t voff = opnd ? (half ? voff_b1 : voff_b) : (half ? voff_a1 : voff_a);
        const uint32_t dst = wave_lds + slot + (opnd ? A_PART + half * B_HALF : half * A_HALF) + j * 4096;
        __builtin_amdgcn_global_load_lds((const DAXQ_GLOBAL void*)(src + voff), (DAXQ_LDS void*)(uintptr_t)dst, 16, 0, 0);
    };
    auto advance = [&]() {
        voff_a += 2 * BKS;
        voff_b += 2 * BKS;
        voff_a1 += 2 * BKS;
        voff_b1 += 2 * BKS;
    };

    const int lr = lane & 15, kg = lane >> 4;
    const int xo = (kg ^ ((lr >> 1) & 3)) << 4;
    const uint8_t* a_rd = smem + (wm * 128 + lr) * BKS + xo;
    const uint8_t* b_rd = smem + A_PART + (wn * 64 + lr) * BKS + xo;
    // fragment f of a pair: 0-7 activation block f, 8-11 weight block f-8; registers 0-3 the first slice, 4-7 the second
    auto read_frag = [&](uint32_t slot, int f, v8i (&af)[NBI], v8i (&bf)[NBJ]) __attribute__((always_inline)) {
        const bool w = f >= NBI;
        const uint8_t* pr = (w ? b_rd + (f - NBI) * 16 * BKS : a_rd + f * 16 * BKS) + slot;
        const v4i lo = *reinterpret_cast<const v4i*>(pr);
        const v4i up = *reinterpret_cast<const v4i*>(pr + (w ? B_HALF : A_HALF));
        const v8i v = __builtin_shufflevector(lo, up, 0, 1, 2, 3, 4, 5, 6, 7);
        if (w) bf[f - NBI] = v;
        else af[f] = v;
    };

    v4f acc[NBJ][NBI];
    v8i fa0[NBI] = {}, fb0[NBJ] = {}, fa1[NBI] = {}, fb1[NBJ] = {};
    auto mfma = [&](auto PAR, auto FIRST, int g) __attribute__((always_inline)) {
        const int j = g / NBI, i = g % NBI;
        const v8i bfr = decltype(PAR)::value ? fb1[j] : fb0[j];
        const v8i afr = decltype(PAR)::value ? fa1[i] : fa0[i];
        if constexpr (decltype(FIRST)::value) {
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

    const int Q = p.k / (2 * BKS);  // pairs; K is a multiple of 128
    uint32_t s0 = 0, s1 = SLOT, s2 = 2 * SLOT;  // slots of pairs q (read a pair ago), q+1, q+2
    // One pair.  PAR: which register set it consumes.  ISSUE: pair q+3 exists, its loads go into the slot of pair q.
    // NEXT: pair q+1 exists, its fragments are read into the other set.  YOUNG: tile loads behind those of pair q+1 that
    // may stay in flight (those of pair q+2).  EXTRA: younger loads that are not tile loads.
    auto pair = [&](auto PAR, auto ISSUE, auto NEXT, auto YOUNG, auto EXTRA, auto FIRST) __attribute__((always_inline)) {
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(YOUNG.value + EXTRA.value) & lgkmcnt0_mask());
        __builtin_amdgcn_s_barrier();  // pair q+1 has landed for everyone, and everyone has read pair q out of its slot
#pragma unroll
        for (int g = 0; g < NREG; ++g) {
            // Two loads per region, the two halves of a 128-byte line: the activation rows' four lines in regions 0, 8,
            // 16, 24, the weight rows' two in regions 4 and 20.  (One load per region in twelve regions, between the
            // regions that read fragments, ran the pair in 0.70 us instead of 0.56: 80.3 against 65.3 us at 1024 x 5120,
            // K = 13824; three or four loads per region 67 to 68 us, all twelve at once 92.7.  The other tiled kernels
            // were tried with their loads in twos as well and are as fast or 1 to 2 % faster with single ones.)
            if constexpr (ISSUE.value) {
                if (g % 8 == 0) {
                    issue_one(s0, g / 4);
                    issue_one(s0, g / 4 + 1);
                } else if (g % 16 == 4) {
                    issue_one(s0, A_LOADS + g / 8);
                    issue_one(s0, A_LOADS + g / 8 + 1);
                }
            }
            if constexpr (NEXT.value) {
                if (g % 2 == 1 && g / 2 < NBI + NBJ) {
                    if constexpr (PAR.value) read_frag(s1, g / 2, fa0, fb0);
                    else read_frag(s1, g / 2, fa1, fb1);
                }
            }
            mfma(PAR, FIRST, g);
            if (g == NREG - 1) {
                if constexpr (ISSUE.value) advance();
                const uint32_t o = s0;
                s0 = s1;
                s1 = s2;
                s2 = o;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    const int tn2 = t & (BN - 1);
    float pre_sx, pre_sw;
    uint32_t pre_b;
    auto request_scales = [&]() __attribute__((always_inline)) {
        pre_sx = p.sx[m0 + t];
        pre_sw = p.sw[n0 + tn2];
        if constexpr (OUTK == DAXQ_F32) pre_b = __float_as_uint((p.bias ? reinterpret_cast<const float*>(p.bias) : p.sw)[n0 + tn2]);
        else pre_b = (p.bias ? p.bias : reinterpret_cast<const uint16_t*>(p.sw))[n0 + tn2];
        __builtin_amdgcn_sched_barrier(0);
    };

    if (Q >= 4) {
        // ---- prologue: pairs 0, 1, 2 in flight (slots s0, s1, s2), pair 0 landed, its fragments in set 0
#pragma unroll
        for (int g = 0; g < PAIR_LOADS; ++g) issue_one(s0, g);
        advance();
#pragma unroll
        for (int g = 0; g < PAIR_LOADS; ++g) issue_one(s1, g);
        advance();
#pragma unroll
        for (int g = 0; g < PAIR_LOADS; ++g) issue_one(s2, g);
        advance();
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(2 * PAIR_LOADS));
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int f = 0; f < NBI + NBJ; ++f) read_frag(s0, f, fa0, fb0);
        // pair 0, then the steady pairs two at a time; the three pairs of the tail are code paths with fixed sets (odd,
        // even, odd after an even number of pairs in front of them, else the fragments move over to the other set once)
        typedef Int<PAIR_LOADS> Y1;
        pair(No{}, Yes{}, Yes{}, Y1{}, Int<0>{}, Yes{});
        int q = 1;
        for (; q + 4 < Q; q += 2) {
            pair(Yes{}, Yes{}, Yes{}, Y1{}, Int<0>{}, No{});
            pair(No{}, Yes{}, Yes{}, Y1{}, Int<0>{}, No{});
        }
        if (q + 3 < Q) {  // one more steady pair: the tail then starts on an even pair, move its fragments to the odd set
            pair(Yes{}, Yes{}, Yes{}, Y1{}, Int<0>{}, No{});
#pragma unroll
            for (int i = 0; i < NBI; ++i) fa1[i] = fa0[i];
#pragma unroll
            for (int j = 0; j < NBJ; ++j) fb1[j] = fb0[j];
        }
        request_scales();
        pair(Yes{}, No{}, Yes{}, Y1{}, Int<3>{}, No{});      // pair Q-3: pairs Q-2 (landing) and Q-1 (in flight)
        pair(No{}, No{}, Yes{}, Int<0>{}, Int<3>{}, No{});   // pair Q-2
        pair(Yes{}, No{}, No{}, Int<0>{}, Int<3>{}, No{});   // pair Q-1
    } else {
        // ---- short K (one to three pairs): load a pair, wait for it, multiply
        request_scales();
        for (int q = 0; q < Q; ++q) {
            if (q) __builtin_amdgcn_s_barrier();
#pragma unroll
            for (int g = 0; g < PAIR_LOADS; ++g) issue_one(0, g);
            advance();
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
            __builtin_amdgcn_s_barrier();
#pragma unroll
            for (int f = 0; f < NBI + NBJ; ++f) read_frag(0, f, fa0, fb0);
            __builtin_amdgcn_s_waitcnt(lgkmcnt0_mask() & vmcnt_imm(63));
            __builtin_amdgcn_sched_barrier(0);
            if (q == 0) {
#pragma unroll
                for (int g = 0; g < NREG; ++g) mfma(No{}, Yes{}, g);
            } else {
#pragma unroll
                for (int g = 0; g < NREG; ++g) mfma(No{}, No{}, g);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    }

    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 7");
#pragma unroll
    for (int j = 0; j < NBJ; ++j)
        asm volatile(""
                     : "+a"(acc[j][0]), "+a"(acc[j][1]), "+a"(acc[j][2]), "+a"(acc[j][3]), "+a"(acc[j][4]), "+a"(acc[j][5]),
                       "+a"(acc[j][6]), "+a"(acc[j][7]));

    __syncthreads();  // every wavefront is past its last fragment read (the short-K loop has no barrier behind its reads)
    tile_epilogue16<DUMP, NBJ, NBI, true, OUTK>(p, acc, smem, m0, n0, t, wm, wn, lr, kg, pre_sx, pre_sw,
                                                !p.bias ? -0.0f : OUTK == DAXQ_F32 ? __uint_as_float(pre_b) : OUTK == DAXQ_F16 ? f16_bits_to_f32((uint16_t)pre_b) : bf16_bits_to_f32(pre_b));
}

}  // namespace daxq
