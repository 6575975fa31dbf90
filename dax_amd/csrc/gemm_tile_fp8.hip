// FP8 W8A8 GEMM on v_mfma_f32_16x16x128_f8f6f4 for gfx950: 256x256 tiles for the large DiT shapes, 128x128 tiles for
// launches with too few of those to fill the CUs.
//
// Every FP8 launch of the tiled kernels goes through this one kernel, so an output element is always the same sequence
// of MFMAs over the same K bytes in the same register positions, whatever tile size, tile order or launch cut it came
// by: a token's FP8 output does not depend on the batch it arrives in.  (The split-K form, gemm_tile256.hip, adds
// partial sums and is documented as differing in the last bits.)
//
// Work decomposition
//   workgroup  BT x BT outputs (BT = 256 or 128), 4 wavefronts (one per SIMD) in a 2 x 2 grid
//   wavefront  BT/2 x BT/2 outputs as NB x NB blocks of 16x16 (NB = 8 or 4), four accumulator registers each
//
// The narrow FP8 MFMA draws less power per operation than the 32x32x64 form (register-only loops on the benchmark's
// values: 4.41 against 4.02 P-op/s).  Its K is 128 bytes, a PAIR of 64-byte slices, and with BT = 256 the operand
// fragments of a pair fill 128 registers, so they cannot all be held twice beside 256 accumulators.  Register plan
// (8 registers per fragment: 16 bytes of either slice of the pair):
//   A (activation rows, MFMA "B" operand)  two sets of NB fragments, the next pair's set read during the odd half
//   B (weight rows, MFMA "A" operand)      ONE set: the MFMAs run B block by B block (j outer, A block i inner), block
//                                          j is dead after its NB MFMAs and is refilled in place for the next pair
//                                          right behind them; the last block, which is in use until the pair ends, has
//                                          a second register set
// LDS: five parts, each ONE operand of ONE pair, [slice of the pair][BT rows][64 B] with the 16-byte chunk swizzle
// chunk ^ ((row >> 1) & 3) (a fragment read takes 16 rows x 4 chunks and is conflict free).  They form a ring in the
// order the loads are issued, ... B(q+1), A(q+1), B(q+2), A(q+2), B(q+3) ...:
//   pair q, even half   MFMAs of the first half of the B blocks; DMA loads of A(q+2) into the part B(q) has left
//   pair q, odd half    MFMAs of the other B blocks; DMA loads of B(q+3) into the part A(q) has left; reads all of A
//                       of pair q+1
// One barrier per half: at the first B(q+1) has landed, at the second A(q+1); every load has two to three slice
// times to land.  Loads are global_load_lds_dwordx4 straight into LDS, addressed as SGPR row-block base + 32-bit lane
// offset, the two halves of a 128-byte line by consecutive instructions.
// A and B of a lane hold the same K bytes (chunk l/16 of the pair's first slice, then of its second), which is all
// the MFMA needs: the order of K inside an instruction is free as long as both operands agree.
// K shorter than four pairs (K < 512) takes a plain loop of the same MFMAs: load a pair, wait, multiply.
#include "gemm_tile.h"
#include "gemm_tile256x128.h"

namespace daxq {

namespace f16 {
constexpr int BKS = 64, T = 256, NPART = 5;
}  // namespace f16

template <bool DUMP, int F8, int BT = 256, int OUTK = DAXQ_BF16>
__device__ __forceinline__ void gemm_tile_fp8_body(const GemmArgs& p, const int block) {
    using namespace f16;
    static_assert(BT == 256 || BT == 128, "tile edge");
    static_assert(OUTK == DAXQ_BF16 || !DUMP, "the accumulator dump exists with bf16 outputs");
    constexpr int NB = BT / 32;             // 16x16 blocks per operand and wavefront
    constexpr int WT = BT / 2;              // edge of a wavefront's outputs
    constexpr int HALF = BT * BKS;          // one slice of one operand: 16 / 8 KB
    constexpr int PART = 2 * HALF;          // one operand of one pair
    constexpr int LPO = BT / 32;            // DMA loads per thread, operand and pair
    constexpr int NREG = NB * NB;           // MFMAs = scheduling regions per pair
    constexpr int HREG = NREG / 2;          // ... per half
    constexpr int DMA_EVERY = HREG / LPO;   // regions per DMA load: 4 / 2
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    int m0, n0;
    if (!tile_origin<BT>(p, block, m0, n0)) return;  // padding slot (before any barrier)

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

    // ---- LDS side: row (w*WT + i*16 + l%16), K chunk l/16 of either slice, stored at chunk (l/16) ^ ((l%16 >> 1) & 3)
    const int lr = lane & 15, kg = lane >> 4;
    const int xo = (kg ^ ((lr >> 1) & 3)) << 4;
    const uint8_t* a_rd = smem + (wm * WT + lr) * BKS + xo;
    const uint8_t* b_rd = smem + (wn * WT + lr) * BKS + xo;
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
    v8i fb[NB - 1];        // B fragments 0 .. NB-2, refilled in place
    v8i fbl_0, fbl_1;      // the last B fragment of even / odd pairs
#pragma clang diagnostic pop

    // MFMA g of a pair: B block g / NB, A block g % NB.  Weights are the MFMA "A" operand (format select cbsz),
    // activations the "B" operand (blgp); accumulators tied in place in AGPRs.
    auto mfma = [&](auto PAR, auto FIRST, int g) __attribute__((always_inline)) {
        constexpr bool par = decltype(PAR)::value;
        const int j = g / NB, i = g % NB;
        const v8i bfr = j == NB - 1 ? (par ? fbl_1 : fbl_0) : fb[j < NB - 1 ? j : 0];
        const v8i afr = par ? fa1[i] : fa0[i];
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
    // the ring, oldest part first: at the start of pair q it holds B(q), A(q) (both read already), B(q+1), A(q+1), B(q+2)
    uint32_t r0 = 0, r1 = PART, r2 = 2 * PART, r3 = 3 * PART, r4 = 4 * PART;

    // One pair of slices.  PAR: parity of the pair (which A set and which last-B set it consumes).
    //   ISSUE_A  pair q+2 exists: its A loads go out during the even half
    //   ISSUE_B  pair q+3 exists: its B loads go out during the odd half
    //   NEXT     pair q+1 exists: read its fragments
    //   EXTRA    younger loads that are not tile loads (the epilogue's scales) and may stay in flight
    //   FIRST    pair 0 of the tile: every block's MFMA starts from zero
    // Region of the odd half (counted from its start) in which A block i of the next pair is read: spread between the B
    // refills, which sit at the multiples of NB.
    auto pair = [&](auto PAR, auto ISSUE_A, auto ISSUE_B, auto NEXT, auto EXTRA, auto FIRST) __attribute__((always_inline)) {
        constexpr bool par = PAR.value, nxt = NEXT.value;
        // ---- even half: B(q+1) has landed; loads younger than it: A(q+1), B(q+2).  The loads of this half overwrite
        // the part that the B fragments of this pair were read from, so every wavefront's reads of it must be over
        // (LDS reads complete in order: all of them are waited for).
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((nxt ? LPO : 0) + (ISSUE_A.value ? LPO : 0) + EXTRA.value) & lgkmcnt0_mask());
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int g = 0; g < NREG; ++g) {
            if (g == HREG) {
                // ---- odd half: A(q+1) has landed; loads younger than it: B(q+2), A(q+2).  (Its loads overwrite the part
                // that this pair's A fragments were read from, a whole half ago: no LDS wait.)
                __builtin_amdgcn_s_waitcnt(vmcnt_imm((ISSUE_A.value ? 2 * LPO : 0) + EXTRA.value));
                __builtin_amdgcn_s_barrier();
            }
            // 128 tiles issue their loads in twos (both halves of a 128-byte line in one region): with a load in every other
            // region of so short a pair nearly every MFMA has a memory instruction in front of it; +2.5 % on launches with
            // a CU per workgroup and long K (512 x 5120 x 5120: 21.0 -> 20.5 us), nothing elsewhere.  The 256 tiles, a
            // load every fourth region, lose 1 % that way.
            constexpr bool twos = BT == 128;
            if constexpr (ISSUE_A.value) {
                if constexpr (twos) {
                    if (g < HREG && g % (2 * DMA_EVERY) == 0) {
                        issue_a(r0, g / DMA_EVERY);
                        issue_a(r0, g / DMA_EVERY + 1);
                    }
                } else {
                    if (g < HREG && g % DMA_EVERY == 0) issue_a(r0, g / DMA_EVERY);
                }
            }
            if constexpr (ISSUE_B.value) {
                if constexpr (twos) {
                    if (g >= HREG && (g - HREG) % (2 * DMA_EVERY) == 0) {
                        issue_b(r1, (g - HREG) / DMA_EVERY);
                        issue_b(r1, (g - HREG) / DMA_EVERY + 1);
                    }
                } else {
                    if (g >= HREG && (g - HREG) % DMA_EVERY == 0) issue_b(r1, (g - HREG) / DMA_EVERY);
                }
            }
            if constexpr (nxt) {
                // the last B block of the next pair into the set this pair does not use
                if (g == (NB == 8 ? 2 : 1)) {
                    if constexpr (par) read_into(fbl_0, b_rd, r2, NB - 1);
                    else read_into(fbl_1, b_rd, r2, NB - 1);
                }
                // B block j right behind its last MFMA of this pair
                if (g >= NB && g % NB == 0) read_into(fb[g / NB - 1], b_rd, r2, g / NB - 1);
                // all of A of the next pair during the odd half, between the B refills
                if (g > HREG) {
                    const int o = g - HREG;  // 1 .. HREG-1
                    int i = -1;
                    if constexpr (NB == 8) {
                        constexpr int at[8] = {1, 4, 7, 10, 13, 15, 18, 21};
#pragma unroll
                        for (int x = 0; x < 8; ++x)
                            if (o == at[x]) i = x;
                    } else {
                        constexpr int at[4] = {1, 2, 3, 5};
#pragma unroll
                        for (int x = 0; x < 4; ++x)
                            if (o == at[x]) i = x;
                    }
                    if (i >= 0) {
                        if constexpr (par) read_into(fa0[i], a_rd, r3, i);
                        else read_into(fa1[i], a_rd, r3, i);
                    }
                }
            }
            mfma(PAR, FIRST, g);
            if constexpr (ISSUE_A.value) {
                if (g == HREG - 2) advance_a();
            }
            if constexpr (ISSUE_B.value) {
                if (g == NREG - 2) advance_b();
            }
            if (g == NREG - 1) {
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

    const float* sxp = p.sx + m0;
    const float* swp = p.sw + n0;
    const int tt = t & (BT - 1);
    float pre_sx, pre_sw;
    uint32_t pre_b;  // the bias element's bits: bf16 / fp16, or fp32
    auto request_scales = [&]() __attribute__((always_inline)) {
        // always three loads per wavefront (a missing bias reads a scale instead and is replaced by -0.0:
        // x + (-0.0) == x bit for bit); with a 128 tile the upper two wavefronts repeat the loads of the lower two
        pre_sx = sxp[tt];
        pre_sw = swp[tt];
        if constexpr (OUTK == DAXQ_F32) pre_b = __float_as_uint((p.bias ? reinterpret_cast<const float*>(p.bias) : p.sw)[n0 + tt]);
        else pre_b = (p.bias ? p.bias : reinterpret_cast<const uint16_t*>(p.sw))[n0 + tt];
        __builtin_amdgcn_sched_barrier(0);
    };

    if (Q >= 4) {
        // ---- prologue: A(0) and B(0) first, then B(1), A(1), B(2) in ring order; fragments of pair 0 into registers
#pragma unroll
        for (int g = 0; g < LPO; ++g) issue_a(r1, g);
        advance_a();
#pragma unroll
        for (int g = 0; g < LPO; ++g) issue_b(r0, g);
        advance_b();
#pragma unroll
        for (int g = 0; g < LPO; ++g) issue_b(r2, g);
        advance_b();
#pragma unroll
        for (int g = 0; g < LPO; ++g) issue_a(r3, g);
        advance_a();
#pragma unroll
        for (int g = 0; g < LPO; ++g) issue_b(r4, g);
        advance_b();
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(3 * LPO));
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int j = 0; j < NB - 1; ++j) read_into(fb[j], b_rd, r0, j);
#pragma unroll
        for (int i = 0; i < NB; ++i) read_into(fa0[i], a_rd, r1, i);
        read_into(fbl_0, b_rd, r0, NB - 1);

        // Pair q consumes register set q % 2 and fills the other one.  Pair 0, then the steady pairs 1 .. Q-4 two at a
        // time (odd, even), then one more if their number is odd.  The three pairs of the tail are code paths of their
        // own with fixed sets (even, odd, even): when the steady pairs end on an even one, the fragments it has read for
        // the next pair are moved over to the even set (once per tile).
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
            fbl_0 = fbl_1;
        }
        pair(No{}, Yes{}, No{}, Yes{}, Int<0>{}, No{});  // pair Q-3 (even): the last A loads

        // the epilogue's scales and bias, requested behind the last tile loads
        request_scales();

        pair(Yes{}, No{}, No{}, Yes{}, Int<3>{}, No{});  // pair Q-2 (odd)
        pair(No{}, No{}, No{}, No{}, Int<3>{}, No{});    // pair Q-1 (even)
    } else {
        // ---- short K (one to three pairs): load a pair, wait for it, multiply.  The same MFMAs on the same fragments
        // as above, so the sums are the same bits as the pipelined path would give.
        request_scales();
        for (int q = 0; q < Q; ++q) {
            if (q) __builtin_amdgcn_s_barrier();  // every wavefront has read pair q-1 out of the two parts
#pragma unroll
            for (int g = 0; g < LPO; ++g) issue_a(r1, g);
#pragma unroll
            for (int g = 0; g < LPO; ++g) issue_b(r0, g);
            advance_a();
            advance_b();
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
            __builtin_amdgcn_s_barrier();
#pragma unroll
            for (int j = 0; j < NB - 1; ++j) read_into(fb[j], b_rd, r0, j);
            read_into(fbl_0, b_rd, r0, NB - 1);
#pragma unroll
            for (int i = 0; i < NB; ++i) read_into(fa0[i], a_rd, r1, i);
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

    // The MFMAs are inline asm, so the compiler cannot count the wait states between one of them and a VALU read of
    // its result: idle cycles first, then every accumulator is passed through an empty statement, which no read of
    // it can move above.
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 7");
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
    tile_epilogue16<DUMP, NB, NB, true, OUTK>(p, acc, smem, m0, n0, t, wm, wn, lr, kg, pre_sx, pre_sw,
                                             !p.bias ? -0.0f : OUTK == DAXQ_F32 ? __uint_as_float(pre_b) : OUTK == DAXQ_F16 ? f16_bits_to_f32((uint16_t)pre_b) : bf16_bits_to_f32(pre_b));
}

template <bool DUMP, int F8, int BT = 256, int OUTK = DAXQ_BF16>
__global__ __launch_bounds__(256) void gemm_tile_fp8_kernel(const GemmArgs p) {
    gemm_tile_fp8_body<DUMP, F8, BT, OUTK>(p, (int)blockIdx.x);
}

// One grid for a launch of few rounds whose left-over tiles run as halves (tail_half_tiles): workgroups 0 .. p.grid - 1
// compute whole 256x256 tiles, the rest the 256x128 halves of the tiles from id quad_base - 1 on.  The halves start on
// the CUs that finish their whole tiles first instead of behind the whole first kernel.
template <bool DUMP, int F8, int OUTK>
__global__ __launch_bounds__(256) void gemm_tile_fp8_then_halves_kernel(const GemmArgs p) {
    if ((int)blockIdx.x < p.grid) gemm_tile_fp8_body<DUMP, F8, 256, OUTK>(p, (int)blockIdx.x);
    else gemm_tile256x128_fp8_body<DUMP, F8, OUTK>(p, (int)blockIdx.x - p.grid);
}

// The same for left-over tiles that run as 128x128 quadrants (tail_tiles): workgroups 0 .. p.grid - 1 compute whole
// tiles, the rest the quadrants of the tiles from id quad_base - 1 on.
template <bool DUMP, int F8, int OUTK>
__global__ __launch_bounds__(256) void gemm_tile_fp8_then_quadrants_kernel(const GemmArgs p) {
    if ((int)blockIdx.x < p.grid) gemm_tile_fp8_body<DUMP, F8, 256, OUTK>(p, (int)blockIdx.x);
    else gemm_tile_fp8_body<DUMP, F8, 128, OUTK>(p, (int)blockIdx.x - p.grid);
}

template <bool DUMP, int F8, int BT, int OUTK>
static int prepare_fp8() {
    static std::atomic<uint64_t> lds_set{0};  // per instantiation
    return ensure_dynamic_lds(reinterpret_cast<const void*>(gemm_tile_fp8_kernel<DUMP, F8, BT, OUTK>), f16::NPART * 2 * BT * f16::BKS, lds_set);
}

template <bool DUMP, int F8, int BT, int OUTK>
static int launch_fp8_impl(const GemmArgs& a, hipStream_t st) {
    if (int rc = prepare_fp8<DUMP, F8, BT, OUTK>()) return rc;
    const int64_t nt = grid_of_order(a);
    if (nt > 0x7fffffff) return fail(DAXQ_ERR_ARG, "gemm: too many tiles");
    hipLaunchKernelGGL((gemm_tile_fp8_kernel<DUMP, F8, BT, OUTK>), dim3((unsigned)nt), dim3(f16::T), f16::NPART * 2 * BT * f16::BKS, st, a);
    return check_launch("gemm_tile_fp8");
}

template <int F8, int BT>
static int launch_fp8_out(const GemmArgs& a, hipStream_t st) {
    if (a.out_kind == DAXQ_F16) return a.acc ? fail(DAXQ_ERR_ARG, "gemm: the accumulator dump exists with bf16 outputs") : launch_fp8_impl<false, F8, BT, DAXQ_F16>(a, st);
    if (a.out_kind == DAXQ_F32) return a.acc ? fail(DAXQ_ERR_ARG, "gemm: the accumulator dump exists with bf16 outputs") : launch_fp8_impl<false, F8, BT, DAXQ_F32>(a, st);
    return a.acc ? launch_fp8_impl<true, F8, BT, DAXQ_BF16>(a, st) : launch_fp8_impl<false, F8, BT, DAXQ_BF16>(a, st);
}

template <int BT>
static int launch_fp8_one(const GemmArgs& a, int f8, hipStream_t st) {
    switch (f8) {
        case 1: return launch_fp8_out<1, BT>(a, st);
        case 2: return launch_fp8_out<2, BT>(a, st);
        case 3: return launch_fp8_out<3, BT>(a, st);
        default: return launch_fp8_out<0, BT>(a, st);
    }
}

// QUADS: the second part of the grid is quadrants (else halves)
template <bool QUADS, bool DUMP, int F8, int OUTK>
static const void* fp8_then_kernel() {
    if constexpr (QUADS) return reinterpret_cast<const void*>(gemm_tile_fp8_then_quadrants_kernel<DUMP, F8, OUTK>);
    else return reinterpret_cast<const void*>(gemm_tile_fp8_then_halves_kernel<DUMP, F8, OUTK>);
}

template <bool QUADS, bool DUMP, int F8, int OUTK>
static int prepare_fp8_then() {
    static std::atomic<uint64_t> lds_set{0};  // per instantiation
    return ensure_dynamic_lds(fp8_then_kernel<QUADS, DUMP, F8, OUTK>(), f16::NPART * 2 * 256 * f16::BKS, lds_set);
}

template <bool QUADS, bool DUMP, int F8, int OUTK>
static int launch_fp8_then_impl(const GemmArgs& a, int64_t nt, hipStream_t st) {
    if (int rc = prepare_fp8_then<QUADS, DUMP, F8, OUTK>()) return rc;
    constexpr int SMEM = f16::NPART * 2 * 256 * f16::BKS;
    if constexpr (QUADS) hipLaunchKernelGGL((gemm_tile_fp8_then_quadrants_kernel<DUMP, F8, OUTK>), dim3((unsigned)nt), dim3(f16::T), SMEM, st, a);
    else hipLaunchKernelGGL((gemm_tile_fp8_then_halves_kernel<DUMP, F8, OUTK>), dim3((unsigned)nt), dim3(f16::T), SMEM, st, a);
    return check_launch(QUADS ? "gemm_tile_fp8_then_quadrants" : "gemm_tile_fp8_then_halves");
}

template <bool QUADS, int F8>
static int launch_fp8_then_out(const GemmArgs& a, int64_t nt, hipStream_t st) {
    if (a.acc && a.out_kind != DAXQ_BF16) return fail(DAXQ_ERR_ARG, "gemm: the accumulator dump exists with bf16 outputs");
    if (a.out_kind == DAXQ_F16) return launch_fp8_then_impl<QUADS, false, F8, DAXQ_F16>(a, nt, st);
    if (a.out_kind == DAXQ_F32) return launch_fp8_then_impl<QUADS, false, F8, DAXQ_F32>(a, nt, st);
    return a.acc ? launch_fp8_then_impl<QUADS, true, F8, DAXQ_BF16>(a, nt, st) : launch_fp8_then_impl<QUADS, false, F8, DAXQ_BF16>(a, nt, st);
}

// `whole` 256x256 tiles of the row-group order, then the pieces of each of the `left` tiles behind them (QUADS: four
// 128x128 quadrants, else two 256x128 halves), in one grid
template <bool QUADS>
static int launch_fp8_then(const GemmArgs& a0, int f8, int whole, int left, hipStream_t st) {
    GemmArgs a = a0;
    a.grid = whole;
    a.quad_base = whole + 1;
    const int64_t nt = (int64_t)whole + (QUADS ? 4 : 2) * (int64_t)left;
    if (nt > 0x7fffffff) return fail(DAXQ_ERR_ARG, "gemm: too many tiles");
    switch (f8) {
        case 1: return launch_fp8_then_out<QUADS, 1>(a, nt, st);
        case 2: return launch_fp8_then_out<QUADS, 2>(a, nt, st);
        case 3: return launch_fp8_then_out<QUADS, 3>(a, nt, st);
        default: return launch_fp8_then_out<QUADS, 0>(a, nt, st);
    }
}

// Every 256x256 tile as its two 256x128 halves (needs m, n >= 256): the grid of launch_fp8_then without whole tiles
int launch_halves_fp8(const GemmArgs& a0, int f8, hipStream_t st) {
    GemmArgs a = a0;
    a.tiles_m = (a.m + 255) / 256;
    a.tiles_n = (a.n + 255) / 256;
    a.order = kOrderRowGroups;
    const int64_t tiles = (int64_t)a.tiles_m * a.tiles_n;
    if (tiles > 0x3fffffff) return fail(DAXQ_ERR_ARG, "gemm: too many tiles");
    return launch_fp8_then<false>(a, f8, 0, (int)tiles, st);
}

// small: 128x128 tiles (needs m, n >= 128); f8: operand formats (kF8XE5 | kF8WE5); tail: the last, partial round of a
// launch of 256x256 tiles as 128x128 quadrants (tail_tiles) or 256x128 halves (tail_half_tiles) in the workgroups
// behind those of the whole tiles -- the same bits either way
int launch_tile_fp8(const GemmArgs& a0, int f8, bool small, int tail, hipStream_t st) {
    GemmArgs a = a0;
    const int bt = small ? 128 : 256;
    a.tiles_m = (a.m + bt - 1) / bt;
    a.tiles_n = (a.n + bt - 1) / bt;
    a.grid = a.quad_base = 0;
    if (small) {
        a.order = kOrderRowGroups;
        return launch_fp8_one<128>(a, f8, st);
    }
    const int left = tail_tiles(a, tail);
    if (left == 0) {
        // more than a quarter and at most half of the CUs' worth of tiles left over: their 256x128 halves with a CU each
        const int halves = tail_half_tiles(a, tail);
        if (halves == 0) return launch_fp8_one<256>(a, f8, st);
        return launch_fp8_then<false>(a, f8, a.tiles_m * a.tiles_n - halves, halves, st);
    }
    return launch_fp8_then<true>(a, f8, a.tiles_m * a.tiles_n - left, left, st);
}

// Every instantiation the launcher can pick, prepared on the current device: afterwards no launch changes a kernel
// attribute any more, so the first launch may already sit inside a stream capture.
int prepare_tile_fp8_kernels() {
    int rc = 0;
#define DAXQ_PREP(...) if (!rc) rc = __VA_ARGS__()
#define DAXQ_PREP_F8(F8)                                  \
    DAXQ_PREP(prepare_fp8<false, F8, 256, DAXQ_BF16>);    \
    DAXQ_PREP(prepare_fp8<true, F8, 256, DAXQ_BF16>);     \
    DAXQ_PREP(prepare_fp8<false, F8, 256, DAXQ_F16>);     \
    DAXQ_PREP(prepare_fp8<false, F8, 256, DAXQ_F32>);     \
    DAXQ_PREP(prepare_fp8<false, F8, 128, DAXQ_BF16>);    \
    DAXQ_PREP(prepare_fp8<true, F8, 128, DAXQ_BF16>);     \
    DAXQ_PREP(prepare_fp8<false, F8, 128, DAXQ_F16>);     \
    DAXQ_PREP(prepare_fp8<false, F8, 128, DAXQ_F32>);     \
    DAXQ_PREP(prepare_fp8_then<false, false, F8, DAXQ_BF16>); \
    DAXQ_PREP(prepare_fp8_then<false, true, F8, DAXQ_BF16>);  \
    DAXQ_PREP(prepare_fp8_then<false, false, F8, DAXQ_F16>);  \
    DAXQ_PREP(prepare_fp8_then<false, false, F8, DAXQ_F32>);  \
    DAXQ_PREP(prepare_fp8_then<true, false, F8, DAXQ_BF16>);  \
    DAXQ_PREP(prepare_fp8_then<true, true, F8, DAXQ_BF16>);   \
    DAXQ_PREP(prepare_fp8_then<true, false, F8, DAXQ_F16>);   \
    DAXQ_PREP(prepare_fp8_then<true, false, F8, DAXQ_F32>)
    DAXQ_PREP_F8(0);
    DAXQ_PREP_F8(1);
    DAXQ_PREP_F8(2);
    DAXQ_PREP_F8(3);
#undef DAXQ_PREP_F8
#undef DAXQ_PREP
    return rc;
}

}  // namespace daxq
