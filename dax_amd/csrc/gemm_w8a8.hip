// W8A8 GEMM on gfx950 MFMA with the fused scale / bias / cast epilogue: the generic kernel (any shape, any
// FP8 operand pairing, bf16 / fp16 / fp32 outputs) and the dispatcher behind the daxq_linear_* entry points.
//
//   INT8: acc[i,j] = sum_k xq[i,k] * wq[j,k]  (int32, exact)   v_mfma_i32_32x32x32_i8
//         out = bf16( f32( bf16( f32_rne(acc) * sx[i] * sw[j] ) ) + f32(bias[j]) )
//         (dax/quant/nn/dynamic/linear.py:214-228: two fp32 multiplies in this order, a
//          bf16 cast, then the bias add as a second bf16 rounding)
//   FP8:  acc = sum_k f32(xq) * f32(wq)       (fp32)           v_mfma_f32_32x32x64_f8f6f4
//         out = bf16( acc * sx[i] * sw[j] + f32(bias[j]) )     (torch._scaled_mm, linear.py:155-173)
//
// Both operands are K-contiguous ([m,k] and [n,k] row-major), which is the layout MFMA
// wants for A and B alike: lane l of a 32x32 MFMA supplies 16 (int8) or 32 (fp8)
// consecutive K bytes of row l%32, K half l/32.  The K order inside an instruction does
// not matter as long as A and B use the same one, and they do.
//
// Tiling: a workgroup owns a BM x BN output tile and walks K in BK-byte slices that are
// double buffered in LDS.  Each 16-byte chunk c of row r sits at chunk slot c ^ f(r) so
// that the ds_read_b128 of 16 consecutive rows at one K offset hits 16 different bank
// groups.  Workgroup ids are remapped so that the tiles resident on one XCD (ids
// congruent mod 8) form a compact patch of the output and share A/B panels in that XCD's L2.
#include <type_traits>

#include "gemm_tile.h"

namespace daxq {

// F8: FP8 operand formats (kF8XE5: the activation bytes, MFMA "A" operand here, are e5m2; kF8WE5: the weight bytes)
template <bool FP8, int BM, int BN, int BK, int WM, int WN, bool DIRECT, int F8 = 0>
__global__ __launch_bounds__(WM* WN * 64) void gemm_w8a8_kernel(const GemmArgs p) {
    constexpr int T = WM * WN * 64;
    constexpr int TM = BM / WM, TN = BN / WN;  // wave tile
    constexpr int MB = TM / 32, NB = TN / 32;  // 32x32 MFMA blocks per wave
    constexpr int CPR = BK / 16;               // 16-byte chunks per tile row
    constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK, STAGE = A_BYTES + B_BYTES;
    constexpr int A_IT = BM * CPR / T, B_IT = BN * CPR / T;
    constexpr int KB = FP8 ? 64 : 32;  // K bytes consumed per MFMA
    constexpr int KSTEPS = BK / KB;
    static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tile must be a multiple of 32x32");
    static_assert((BM * CPR) % T == 0 && (BN * CPR) % T == 0, "tile chunks must divide over the threads");
    static_assert(CPR == 8, "swizzle is written for 128-byte tile rows");
    typedef typename AccT<FP8>::type acc_t;

    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave / WN, wn = wave % WN;
    int tm, tn;
    tile_of_block(p.gm, blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

    // ---- global -> LDS mapping: chunk g = j*T + t -> tile row g/8, LDS slot g%8, global chunk slot^f(row)
    const uint8_t* ga[A_IT];
    const uint8_t* gb[B_IT];
    int la[A_IT], lb[B_IT];
#pragma unroll
    for (int j = 0; j < A_IT; ++j) {
        const int g = j * T + t, row = g >> 3, slot = g & 7;
        int gr = m0 + row;
        gr = gr < p.m ? gr : p.m - 1;
        ga[j] = p.a + (int64_t)gr * p.lda + ((slot ^ swz(row)) << 4);
        la[j] = g << 4;
    }
#pragma unroll
    for (int j = 0; j < B_IT; ++j) {
        const int g = j * T + t, row = g >> 3, slot = g & 7;
        int gr = n0 + row;
        gr = gr < p.n ? gr : p.n - 1;
        gb[j] = p.b + (int64_t)gr * p.ldb + ((slot ^ swz(row)) << 4);
        lb[j] = A_BYTES + (g << 4);
    }

    // ---- LDS -> MFMA operand mapping
    const int l31 = lane & 31, hi = lane >> 5;
    const int fl = swz(l31);
    const int a_row_off = (wm * TM + l31) * BK;
    const int b_row_off = A_BYTES + (wn * TN + l31) * BK;

    acc_t acc[MB][NB];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

    const int KT = p.k / BK;

    auto compute = [&](int stage) {
        const uint8_t* base = smem + stage * STAGE;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            if constexpr (!FP8) {
                const int xo = (((ks * 2 + hi) ^ fl) << 4);
                v4i af[MB], bf[NB];
#pragma unroll
                for (int i = 0; i < MB; ++i) af[i] = *reinterpret_cast<const v4i*>(base + a_row_off + i * 32 * BK + xo);
#pragma unroll
                for (int j = 0; j < NB; ++j) bf[j] = *reinterpret_cast<const v4i*>(base + b_row_off + j * 32 * BK + xo);
#pragma unroll
                for (int i = 0; i < MB; ++i)
#pragma unroll
                    for (int j = 0; j < NB; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
            } else {
                const int xo0 = (((ks * 4 + hi * 2) ^ fl) << 4);
                const int xo1 = (((ks * 4 + hi * 2 + 1) ^ fl) << 4);
                v8i af[MB], bf[NB];
#pragma unroll
                for (int i = 0; i < MB; ++i) {
                    v4i lo = *reinterpret_cast<const v4i*>(base + a_row_off + i * 32 * BK + xo0);
                    v4i hi4 = *reinterpret_cast<const v4i*>(base + a_row_off + i * 32 * BK + xo1);
                    af[i] = __builtin_shufflevector(lo, hi4, 0, 1, 2, 3, 4, 5, 6, 7);
                }
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    v4i lo = *reinterpret_cast<const v4i*>(base + b_row_off + j * 32 * BK + xo0);
                    v4i hi4 = *reinterpret_cast<const v4i*>(base + b_row_off + j * 32 * BK + xo1);
                    bf[j] = __builtin_shufflevector(lo, hi4, 0, 1, 2, 3, 4, 5, 6, 7);
                }
#pragma unroll
                for (int i = 0; i < MB; ++i)
#pragma unroll
                    for (int j = 0; j < NB; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[i], bf[j], acc[i][j], (F8 & kF8XE5) ? 1 : 0, (F8 & kF8WE5) ? 1 : 0, 0, 0, 0, 0);
            }
        }
    };

    if constexpr (DIRECT) {
        // global_load_lds_dwordx4: each wavefront instruction drops 64 consecutive 16-byte
        // chunks into LDS at a wave-uniform base; the swizzle lives in the global address.
        auto issue = [&](int kt, int stage) {
            const int koff = kt * BK;
            uint8_t* sbase = smem + stage * STAGE;
#pragma unroll
            for (int j = 0; j < A_IT; ++j)
                __builtin_amdgcn_global_load_lds((const DAXQ_GLOBAL void*)(ga[j] + koff),
                                                 (DAXQ_LDS void*)(sbase + ((j * T + wave * 64) << 4)), 16, 0, 0);
#pragma unroll
            for (int j = 0; j < B_IT; ++j)
                __builtin_amdgcn_global_load_lds((const DAXQ_GLOBAL void*)(gb[j] + koff),
                                                 (DAXQ_LDS void*)(sbase + A_BYTES + ((j * T + wave * 64) << 4)), 16, 0, 0);
        };
        issue(0, 0);
        for (int kt = 0; kt < KT; ++kt) {
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
            __syncthreads();
            if (kt + 1 < KT) issue(kt + 1, (kt + 1) & 1);
            compute(kt & 1);
        }
    } else {
        uint4 ra[A_IT], rb[B_IT];
        auto gload = [&](int kt) {
            const int koff = kt * BK;
#pragma unroll
            for (int j = 0; j < A_IT; ++j) ra[j] = *reinterpret_cast<const uint4*>(ga[j] + koff);
#pragma unroll
            for (int j = 0; j < B_IT; ++j) rb[j] = *reinterpret_cast<const uint4*>(gb[j] + koff);
        };
        auto lstore = [&](int stage) {
            uint8_t* sbase = smem + stage * STAGE;
#pragma unroll
            for (int j = 0; j < A_IT; ++j) *reinterpret_cast<uint4*>(sbase + la[j]) = ra[j];
#pragma unroll
            for (int j = 0; j < B_IT; ++j) *reinterpret_cast<uint4*>(sbase + lb[j]) = rb[j];
        };
        gload(0);
        lstore(0);
        __syncthreads();
        for (int kt = 0; kt < KT; ++kt) {
            if (kt + 1 < KT) gload(kt + 1);
            compute(kt & 1);
            if (kt + 1 < KT) lstore((kt + 1) & 1);
            __syncthreads();
        }
    }

    // ---- epilogue: lane owns column n = l%32 of each 32x32 block, register v owns row
    //      8*(v/4) + 4*(l/32) + v%4.  The element type of out / bias is a run-time choice here (this kernel is the
    //      one that serves fp16 / fp32 modules): INT8 rounds to that type, then adds the bias in it (a second
    //      rounding, dax/quant/nn/dynamic/linear.py:225-228); FP8 adds the bias in fp32 and rounds once (_scaled_mm).
    auto epilogue = [&](auto KIND) {
        constexpr int OK = decltype(KIND)::value;
        auto round_out = [](float y) -> float {  // y rounded to the output type, as a float
            if constexpr (OK == DAXQ_BF16) {
                return bf16_bits_to_f32(f32_to_bf16_bits(y));
            } else if constexpr (OK == DAXQ_F16) {
                // The empty statement hides where y comes from.  Without it the instruction selector folds the fp32
                // multiply (or add) that produced y and this conversion into one mixed-precision fma
                // (v_fma_mixlo_f16), which rounds the exact product ONCE to fp16: on products whose fp32 rounding
                // lands on an fp16 tie that is a different result from the two roundings the op sequence asks for.
                asm volatile("" : "+v"(y));
                return (float)(_Float16)y;
            } else {
                return y;
            }
        };
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            const int n = n0 + wn * TN + j * 32 + l31;
            const bool n_ok = n < p.n;
            const int nc = n_ok ? n : p.n - 1;
            const float swv = p.sw[nc];
            float bv = 0.0f;
            if (p.bias) {
                if constexpr (OK == DAXQ_BF16) bv = bf16_bits_to_f32(p.bias[nc]);
                else if constexpr (OK == DAXQ_F16) bv = (float)reinterpret_cast<const _Float16*>(p.bias)[nc];
                else bv = reinterpret_cast<const float*>(p.bias)[nc];
            }
#pragma unroll
            for (int i = 0; i < MB; ++i) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int m = m0 + wm * TM + i * 32 + 8 * (v >> 2) + 4 * hi + (v & 3);
                    if (m < p.m && n_ok) {
                        const float sxv = p.sx[m];
                        float o;
                        if constexpr (!FP8) {
                            float y = (float)acc[i][j][v];  // v_cvt_f32_i32, round to nearest even
                            y = y * sxv;
                            y = y * swv;
                            o = round_out(y);
                            if (p.bias) o = round_out(o + bv);
                            if (p.acc) static_cast<int32_t*>(p.acc)[(int64_t)m * p.ldacc + n] = acc[i][j][v];
                        } else {
                            o = round_out(acc[i][j][v] * sxv * swv + bv);
                            if (p.acc) static_cast<float*>(p.acc)[(int64_t)m * p.ldacc + n] = acc[i][j][v];
                        }
                        const int64_t at = (int64_t)m * p.ldo + n;
                        if constexpr (OK == DAXQ_BF16) p.out[at] = (uint16_t)(__float_as_uint(o) >> 16);
                        else if constexpr (OK == DAXQ_F16) reinterpret_cast<_Float16*>(p.out)[at] = (_Float16)o;
                        else reinterpret_cast<float*>(p.out)[at] = o;
                    }
                }
            }
        }
    };
    if (p.out_kind == DAXQ_BF16) epilogue(std::integral_constant<int, DAXQ_BF16>{});
    else if (p.out_kind == DAXQ_F16) epilogue(std::integral_constant<int, DAXQ_F16>{});
    else epilogue(std::integral_constant<int, DAXQ_F32>{});
}

bool tile256_applies(const GemmArgs& a);
int launch_tile_i8(const GemmArgs& a, bool small, int tail, hipStream_t st);           // gemm_tile256.hip
int launch_tile_fp8(const GemmArgs& a, int f8, bool small, int tail, hipStream_t st);  // gemm_tile_fp8.hip
int launch_halves_i8(const GemmArgs& a, hipStream_t st);                                // gemm_tile256.hip
int launch_halves_fp8(const GemmArgs& a, int f8, hipStream_t st);                       // gemm_tile_fp8.hip
template <bool FP8>
int launch_tile128_splitk(const GemmArgs& a, int f8, hipStream_t st);

template <bool FP8>
static int launch_tiled(const GemmArgs& a, int f8, bool small, int tail, hipStream_t st) {
    if constexpr (FP8) return launch_tile_fp8(a, f8, small, tail, st);
    else return launch_tile_i8(a, small, tail, st);
}

template <bool FP8>
static int launch_halves(const GemmArgs& a, int f8, hipStream_t st) {
    if constexpr (FP8) return launch_halves_fp8(a, f8, st);
    else return launch_halves_i8(a, st);
}

int prepare_tile_fp8_kernels();
int prepare_tile256_kernels();

template <bool FP8, int BM, int BN, int BK, int WM, int WN, bool DIRECT, int F8 = 0>
static int prepare_cfg() {
    static std::atomic<uint64_t> lds_set{0};  // per instantiation
    return ensure_dynamic_lds(reinterpret_cast<const void*>(gemm_w8a8_kernel<FP8, BM, BN, BK, WM, WN, DIRECT, F8>),
                              2 * (BM + BN) * BK, lds_set);
}

template <bool FP8, int BM, int BN, int BK, int WM, int WN, bool DIRECT, int F8 = 0>
static int launch_cfg(const GemmArgs& a0, hipStream_t st) {
    GemmArgs a = a0;
    a.tiles_m = (a.m + BM - 1) / BM;
    a.tiles_n = (a.n + BN - 1) / BN;
    constexpr int smem = 2 * (BM + BN) * BK;
    auto kern = gemm_w8a8_kernel<FP8, BM, BN, BK, WM, WN, DIRECT, F8>;
    if (int rc = prepare_cfg<FP8, BM, BN, BK, WM, WN, DIRECT, F8>()) return rc;
    const int64_t nt = (int64_t)a.tiles_m * a.tiles_n;
    if (nt > 0x7fffffff) return fail(DAXQ_ERR_ARG, "gemm: too many tiles");
    hipLaunchKernelGGL(kern, dim3((unsigned)nt), dim3(WM * WN * 64), smem, st, a);
    return check_launch("gemm_w8a8");
}

// the generic kernel on BT x BT tiles for any FP8 operand pairing
template <bool FP8, int BT>
static int launch_generic(const GemmArgs& a, int f8, hipStream_t st) {
    constexpr int WN = BT == 256 ? 4 : 2;
    if constexpr (FP8) {
        switch (f8) {
            case 1: return launch_cfg<true, BT, BT, 128, 2, WN, true, 1>(a, st);
            case 2: return launch_cfg<true, BT, BT, 128, 2, WN, true, 2>(a, st);
            case 3: return launch_cfg<true, BT, BT, 128, 2, WN, true, 3>(a, st);
            default: break;
        }
    }
    return launch_cfg<FP8, BT, BT, 128, 2, WN, true, 0>(a, st);
}

// Kernel choices of the `kernel` argument (daxq_linear_w8a8): low 16 bits pick the implementation, bits 16-23 the
// depth of the tile-order groups (0 = 4 tile rows).
enum { K_DEFAULT = 0, K_GENERIC256 = 2, K_GENERIC128 = 5, K_TILED_256 = 8, K_TILED_128 = 11, K_TILED_HALVES = 14 };

// Tile order a launch of 256x256 tiles takes when the caller names none.  The banded order (tile_order.h: patches of
// 8 x 4 tiles per XCD, the eight XCDs of a round on the same activation rows and on different weight bands) reads the
// least from the L2s' far side and was the fastest order on every large shape measured (INT8 and FP8 alike; M = 20000
// to 75600, among them every second tile row from 63488 up; K = 2048 to 13824; N = 5120 to 15360: +0.6 to +5.8 % over
// the row groups, most at long K, and none of the row groups' 3-4 % dips where the XCD ranges start on the same
// columns).  It deals whole patches of 32 tiles to the XCDs, so one XCD can end up with more tiles than an eighth of
// them: it is taken when the slowest XCD needs at most 5 % more tile times than the row groups do; with fewer than
// five bands (N < 5120), K below 2048 or few rounds the row groups were as fast or faster (K = 1536: -2 %; N = K = 4096:
// -2 %; M = 9450, a 1/8 share of the rows, 3 to 9 rounds: -0.8 to +2 % per linear and +0.2 / +1.0 % INT8 / FP8 over the
// four, now that the rows under the last whole step form dense patches, -3 to -16 % before; M = 4725: -4 to -5 %; M =
// 20000: +3 % at N >= 13824, -3 % at N = 5120, where the row groups run their last tiles as quadrants).
static int order_by_shape(int64_t m, int64_t n, int64_t k) {
    const int64_t tm = (m + 255) / 256, tn = (n + 255) / 256, tiles = tm * tn;
    // (tm >= 64: at least two super-rows of whole 8 x 4 patches; tm <= 100000 and tn <= 4096: the range the host-side
    // coverage check of the order reaches, with sampled grids)
    if (k < 2048 || tn < 20 || tm < 64 || tiles < 2048 || tm > 100000 || tn > 4096) return kOrderRowGroups;
    return banded_xcd_rounds((int)tm, (int)tn, 4) * 100 <= (tiles + 255) / 256 * 105 ? kOrderBanded : kOrderRowGroups;
}

template <bool FP8>
static int launch_gemm(const void* xq, int64_t ld_xq, const float* sx, const void* wq, int64_t ld_wq, const float* sw,
                       const void* bias, void* out, int64_t ld_out, void* acc, int64_t ld_acc, int64_t m, int64_t n,
                       int64_t k, hipStream_t st, int f8 = 0, int out_kind = DAXQ_BF16, int kernel = 0) {
    if (m < 0 || n < 0 || k <= 0 || ld_xq < k || ld_wq < k || ld_out < n || (acc && ld_acc < n))
        return fail(DAXQ_ERR_ARG, "linear: bad shape m=%lld n=%lld k=%lld", (long long)m, (long long)n, (long long)k);
    if (out_kind != DAXQ_BF16 && out_kind != DAXQ_F16 && out_kind != DAXQ_F32) return fail(DAXQ_ERR_ARG, "linear: unknown output type %d", out_kind);
    if (m == 0 || n == 0) return DAXQ_OK;
    if (!xq || !sx || !wq || !sw || !out) return fail(DAXQ_ERR_ARG, "linear: null pointer");
    if (m > 0x7fffffff || n > 0x7fffffff || k > 0x7fffffff) return fail(DAXQ_ERR_ARG, "linear: dimension exceeds int32");
    if (k % DAXQ_K_ALIGN != 0) return fail(DAXQ_ERR_ALIGN, "linear: k=%lld is not a multiple of %d (zero-pad the operands)", (long long)k, DAXQ_K_ALIGN);
    if (((uintptr_t)xq & 15) || ((uintptr_t)wq & 15) || (ld_xq & 15) || (ld_wq & 15))
        return fail(DAXQ_ERR_ALIGN, "linear: xq/wq must be 16-byte aligned with leading dimensions that are multiples of 16");
    const uintptr_t oa = out_kind == DAXQ_F32 ? 3 : 1;
    if (((uintptr_t)out & oa) || ((uintptr_t)sx & 3) || ((uintptr_t)sw & 3) || ((uintptr_t)bias & oa) || ((uintptr_t)acc & 3))
        return fail(DAXQ_ERR_ALIGN, "linear: misaligned out/scale/bias/acc pointer");
    GemmArgs a;
    a.a = static_cast<const uint8_t*>(xq);
    a.b = static_cast<const uint8_t*>(wq);
    a.sx = sx;
    a.sw = sw;
    a.bias = static_cast<const uint16_t*>(bias);
    a.out = static_cast<uint16_t*>(out);
    a.acc = acc;
    a.lda = ld_xq;
    a.ldb = ld_wq;
    a.ldo = ld_out;
    a.ldacc = ld_acc;
    a.m = (int)m;
    a.n = (int)n;
    a.k = (int)k;
    a.tiles_m = a.tiles_n = 0;
    a.gm = (kernel >> 16) & 0xff ? (kernel >> 16) & 0xff : 4;
    // Tile order of the 256x256 kernels: bits 24-27 of `kernel`, 0 = by shape (order_by_shape), 1 = groups of tile rows,
    // 2 = banded
    const int order_bits = (kernel >> 24) & 15;
    if (order_bits > 2) return fail(DAXQ_ERR_ARG, "linear: unknown tile order %d", order_bits);
    a.order = order_bits ? order_bits - 1 : order_by_shape(m, n, k);
    a.out_kind = out_kind;
    a.splits = 1;
    a.counters = nullptr;
    a.partials = nullptr;
    a.grid = a.quad_base = 0;
    // bits 28-29 of `kernel`: the last partial round of a launch of 256x256 tiles as 128x128 quadrants (or, when its tiles
    // number more than a quarter of the CUs, as 256x128 halves): 0 = by shape, 1 = never, 2 = whenever every piece gets a CU of its own
    const int tail = (kernel >> 28) & 3;
    if (tail > 2) return fail(DAXQ_ERR_ARG, "linear: unknown tail choice %d", tail);
    const int which = kernel & 0xffff;
    const bool fits32 = a.lda < (1 << 26) && a.ldb < (1 << 26);  // 32-bit row offsets of the tiled kernels
    if (acc && out_kind != DAXQ_BF16 && which != K_GENERIC256 && which != K_GENERIC128 && which != K_DEFAULT)
        return fail(DAXQ_ERR_ARG, "linear: the tiled kernels dump their accumulators with bf16 outputs only");
    switch (which) {
        case K_DEFAULT: {
            // fp16 / fp32 outputs together with the accumulator dump (tests): the generic kernel
            if (acc && out_kind != DAXQ_BF16)
                return (m >= 256 && n >= 256) ? launch_generic<FP8, 256>(a, f8, st) : launch_generic<FP8, 128>(a, f8, st);
            // library default: the tiled kernel on 256x256 tiles once there is one for every second CU, on 128x128
            // tiles (4x as many workgroups, two per CU) below that, and the generic kernel for operands smaller than
            // one such tile.  Measured at N = K = 5120 (INT8, T-op/s, 128 / 256 tiles):
            // M = 512 -> 1127 / 551, M = 1024 (80 large tiles) -> 1275 / 1055, M = 2048 (160) -> 1542 / 1817;
            // 4096 x 1536 x 1536 (96) -> 1182 / 895, 8192 x 1536 x 1536 (192) -> 1517 / 1587.
            // Between a quarter and a half of the CUs' worth of large tiles, every tile runs as its two 256x128 halves with
            // a CU each (K >= 2048).  Measured against what these launches took before (128x128 tiles up to 127 large
            // tiles, whole 256x256 tiles at 128), INT8 / e4m3, us: 1024 x 5120 x 5120 (80 tiles) 38.7 -> 31.0 / 37.7 -> 29.6,
            // 1536 x 5120 x 5120 (120) 41.1 -> 35.0 / 40.3 -> 35.3, 1100 x 4352 x 5120 (85) 42.4 -> 31.6 / 41.1 -> 31.1,
            // 2048 x 4096 x 4096 (128) 39.6 -> 30.7 / 38.7 -> 31.2, 1024 x 5120, K = 13824 95.9 -> 69.3 / 93.1 -> 66.8,
            // 4096 x 1536, K = 8960 62.3 -> 50.7 / 60.5 -> 50.3, K = 3072 +9 to +15 % / +16 %, K = 2048 0 to +10 % / +2 %;
            // at K = 1536 -2 / -5 %, and with 60 tiles (768 x 5120 x 5120) the quadrants' 23.8 us become 30.5.
            const int64_t tiles256 = ((m + 255) / 256) * ((n + 255) / 256);
            const int cus = cu_count();
            if (tile256_applies(a) && k >= 2048 && cus >= 8 && 4 * tiles256 > cus && 2 * tiles256 <= cus) return launch_halves<FP8>(a, f8, st);
            if (tile256_applies(a) && tiles256 >= 128) return launch_tiled<FP8>(a, f8, false, tail, st);
            if (m >= 128 && n >= 128 && fits32) return launch_tiled<FP8>(a, f8, true, 1, st);
            return launch_generic<FP8, 128>(a, f8, st);
        }
        case K_GENERIC256: return launch_generic<FP8, 256>(a, f8, st);
        case K_GENERIC128: return launch_generic<FP8, 128>(a, f8, st);
        case K_TILED_256:
            if (!tile256_applies(a)) return fail(DAXQ_ERR_ARG, "linear: the 256x256 kernel needs m, n >= 256");
            return launch_tiled<FP8>(a, f8, false, tail, st);
        case K_TILED_128:
            if (m < 128 || n < 128 || !fits32) return fail(DAXQ_ERR_ARG, "linear: the 128x128 kernel needs m, n >= 128");
            return launch_tiled<FP8>(a, f8, true, 1, st);
        case K_TILED_HALVES:
            if (!tile256_applies(a)) return fail(DAXQ_ERR_ARG, "linear: the 256x128 kernel needs m, n >= 256");
            return launch_halves<FP8>(a, f8, st);
        default: return fail(DAXQ_ERR_ARG, "linear: unknown kernel choice %d", which);
    }
}

// ---- split-K: launches with too few 128x128 tiles to fill the CUs cut K into ranges ------------------------------
constexpr int64_t kPartialBytes = 128 * 128 * 4;  // one workgroup's accumulators: 64 registers x 256 lanes

static int64_t splitk_tiles(int64_t m, int64_t n) { return ((m + 127) / 128) * ((n + 127) / 128); }
// The head of a workspace holds the tile counters.  Its size is fixed, not derived from the problem: a workspace is
// reused by launches of different shapes, and the counters must stay zero between them, so no launch may ever put
// partial results where another one keeps counters.
constexpr int64_t kCounterBytes = 16384;
constexpr int64_t kMaxSplitTiles = kCounterBytes / 4;

// How many ranges pay: as many as give every workgroup a CU of its own (tiles x ranges <= 256), keep a range at
// least 1024 bytes of K deep and divide K / 128 evenly; 1 = no split.  Measured at N = K = 5120 (INT8, us, plain launch /
// 2 / 4 ranges): M = 256 (80 tiles) 34 / 28 / 40, M = 512 (160 tiles) 24 / 35 / 52, M = 1024 52 / 71 / -: the partial
// results make a round trip through device-coherent memory (about 10 us for 20 MB), which only idle CUs pay for.
static int splitk_choice(int64_t m, int64_t n, int64_t k) {
    if (m < 128 || n < 128 || k % DAXQ_K_ALIGN) return 1;
    const int64_t tiles = splitk_tiles(m, n), units = k / DAXQ_K_ALIGN;
    int best = 1;
    for (int s = 2; s <= 8; ++s)
        if (units % s == 0 && k / s >= 1024 && tiles * s <= 256) best = s;
    return best;
}

template <bool FP8>
static int launch_gemm_splitk(const void* xq, int64_t ld_xq, const float* sx, const void* wq, int64_t ld_wq,
                              const float* sw, const void* bias, void* out, int64_t ld_out, int64_t m, int64_t n, int64_t k,
                              int splits, void* workspace, int64_t workspace_bytes, hipStream_t st, int f8) {
    if (splits == 0) splits = splitk_choice(m, n, k);
    if (splits <= 1)  // nothing to split (or not worth it): the plain launch, which needs no workspace
        return launch_gemm<FP8>(xq, ld_xq, sx, wq, ld_wq, sw, bias, out, ld_out, nullptr, 0, m, n, k, st, f8);
    if (m < 128 || n < 128) return fail(DAXQ_ERR_ARG, "linear_splitk: needs m, n >= 128 (got %lld, %lld)", (long long)m, (long long)n);
    if (m > 0x7fffffff || n > 0x7fffffff || k <= 0 || k > 0x7fffffff || ld_xq < k || ld_wq < k || ld_out < n)
        return fail(DAXQ_ERR_ARG, "linear_splitk: bad shape m=%lld n=%lld k=%lld", (long long)m, (long long)n, (long long)k);
    if (k % DAXQ_K_ALIGN != 0 || (k / DAXQ_K_ALIGN) % splits != 0)
        return fail(DAXQ_ERR_ALIGN, "linear_splitk: k=%lld does not divide into %d ranges that are multiples of %d", (long long)k, splits, DAXQ_K_ALIGN);
    if (!xq || !sx || !wq || !sw || !out) return fail(DAXQ_ERR_ARG, "linear_splitk: null pointer");
    if (((uintptr_t)xq & 15) || ((uintptr_t)wq & 15) || (ld_xq & 15) || (ld_wq & 15) || ld_xq >= (1 << 26) || ld_wq >= (1 << 26))
        return fail(DAXQ_ERR_ALIGN, "linear_splitk: xq/wq must be 16-byte aligned with leading dimensions that are multiples of 16 below 2^26");
    if (((uintptr_t)out & 1) || ((uintptr_t)sx & 3) || ((uintptr_t)sw & 3) || ((uintptr_t)bias & 1))
        return fail(DAXQ_ERR_ALIGN, "linear_splitk: misaligned out/scale/bias pointer");
    const int64_t tiles = splitk_tiles(m, n), cbytes = kCounterBytes;
    if (tiles > kMaxSplitTiles) return fail(DAXQ_ERR_ARG, "linear_splitk: %lld output tiles, at most %lld (split-K is for launches with few tiles)", (long long)tiles, (long long)kMaxSplitTiles);
    const int64_t need = cbytes + tiles * splits * kPartialBytes;
    if (!workspace || ((uintptr_t)workspace & 255)) return fail(DAXQ_ERR_ALIGN, "linear_splitk: the workspace must be 256-byte aligned");
    if (workspace_bytes < need)
        return fail(DAXQ_ERR_ARG, "linear_splitk: workspace of %lld bytes, %lld needed for m=%lld n=%lld in %d ranges", (long long)workspace_bytes,
                    (long long)need, (long long)m, (long long)n, splits);
    GemmArgs a;
    a.a = static_cast<const uint8_t*>(xq);
    a.b = static_cast<const uint8_t*>(wq);
    a.sx = sx;
    a.sw = sw;
    a.bias = static_cast<const uint16_t*>(bias);
    a.out = static_cast<uint16_t*>(out);
    a.acc = nullptr;
    a.lda = ld_xq;
    a.ldb = ld_wq;
    a.ldo = ld_out;
    a.ldacc = 0;
    a.m = (int)m;
    a.n = (int)n;
    a.k = (int)k;
    a.tiles_m = a.tiles_n = 0;
    a.gm = 4;
    a.order = 0;
    a.out_kind = DAXQ_BF16;
    a.splits = splits;
    a.grid = a.quad_base = 0;
    a.counters = static_cast<int32_t*>(workspace);
    a.partials = static_cast<uint8_t*>(workspace) + cbytes;
    return launch_tile128_splitk<FP8>(a, f8, st);
}

static int splitk_formats(int x_fmt, int w_fmt, bool& fp8, int& f8) {
    const bool x8 = x_fmt == DAXQ_FMT_E4M3 || x_fmt == DAXQ_FMT_E5M2, w8 = w_fmt == DAXQ_FMT_E4M3 || w_fmt == DAXQ_FMT_E5M2;
    if (x_fmt == DAXQ_FMT_I8 && w_fmt == DAXQ_FMT_I8) {
        fp8 = false;
        f8 = 0;
        return DAXQ_OK;
    }
    if (x8 && w8) {
        fp8 = true;
        f8 = (x_fmt == DAXQ_FMT_E5M2 ? kF8XE5 : 0) | (w_fmt == DAXQ_FMT_E5M2 ? kF8WE5 : 0);
        return DAXQ_OK;
    }
    return fail(DAXQ_ERR_ARG, "linear: unsupported operand formats x=%d w=%d (int8 x int8, or fp8 x fp8)", x_fmt, w_fmt);
}

// ---- split-K on the library's own scratch memory (for callers that cannot allocate) ------------------------------
// The workspace of daxq_linear_w8a8_splitk as a file-scope device array: tile counters at its head, then room for 512
// partial results of 64 KiB (tiles x ranges <= 512; splitk_choice never asks for more than 256).  Every
// device the library runs on holds its own copy at its own address until the process ends.  `scratch` is only the
// host-side handle of the array: host code uses the per-device address that hipGetSymbolAddress returned, never the name.
constexpr int64_t kStaticSlots = 512;
constexpr int64_t kStaticScratchBytes = kCounterBytes + kStaticSlots * kPartialBytes;
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];      // device address of `scratch`, per device
// The counters at the head of the array need no clearing: a file-scope device array is zero when the code object is
// loaded, and every launch leaves the counters it used at zero.

// Address of the current device's copy of `scratch`, looked up once per device.
static int scratch_of_current_device(void** ptr, int* dev_out) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return fail(DAXQ_ERR_LAUNCH, "hipGetDevice failed");
    if (dev < 0 || dev >= kMaxDevices) return fail(DAXQ_ERR_DEVICE, "linear_splitk_static: device index %d, at most %d devices", dev, kMaxDevices);
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return fail(DAXQ_ERR_LAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
        if ((uintptr_t)p & 255) return fail(DAXQ_ERR_ALIGN, "the library's scratch array is not 256-byte aligned on device %d", dev);
        g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *ptr = p;
    *dev_out = dev;
    return DAXQ_OK;
}

}  // namespace daxq

extern "C" {

int daxq_linear_w8a8_splitk_static(int x_fmt, int w_fmt, const void* xq, int64_t ld_xq, const float* sx, const void* wq,
                                   int64_t ld_wq, const float* sw, const void* bias, void* out, int64_t ld_out,
                                   int64_t m, int64_t n, int64_t k, int splits, daxq_stream_t stream) {
    using namespace daxq;
    bool fp8;
    int f8;
    if (int rc = splitk_formats(x_fmt, w_fmt, fp8, f8)) return rc;
    if (splits < 0 || splits > 64) return fail(DAXQ_ERR_ARG, "linear_splitk_static: splits must be 0 (library's choice) to 64");
    if (m < 0 || n < 0 || k <= 0) return fail(DAXQ_ERR_ARG, "linear_splitk_static: bad shape m=%lld n=%lld k=%lld", (long long)m, (long long)n, (long long)k);
    if (splits == 0) splits = splitk_choice(m, n, k);
    hipStream_t st = (hipStream_t)stream;
    void* ws = nullptr;
    if (splits > 1) {
        const int64_t slots = splitk_tiles(m, n) * splits;
        if (slots > kStaticSlots)
            return fail(DAXQ_ERR_ARG, "linear_splitk_static: %lld output tiles of 128x128 in %d ranges need %lld partial results, the library's "
                        "scratch array holds %lld (%lld bytes); use daxq_linear_w8a8_splitk with a workspace", (long long)splitk_tiles(m, n),
                        splits, (long long)slots, (long long)kStaticSlots, (long long)kStaticScratchBytes);
        int dev = 0;
        if (int rc = scratch_of_current_device(&ws, &dev)) return rc;
    }
    return fp8 ? launch_gemm_splitk<true>(xq, ld_xq, sx, wq, ld_wq, sw, bias, out, ld_out, m, n, k, splits, ws,
                                          kStaticScratchBytes, st, f8)
               : launch_gemm_splitk<false>(xq, ld_xq, sx, wq, ld_wq, sw, bias, out, ld_out, m, n, k, splits, ws,
                                           kStaticScratchBytes, st, 0);
}

int daxq_linear_splitk_choice(int64_t m, int64_t n, int64_t k) { return daxq::splitk_choice(m, n, k); }

int daxq_linear_tile_order_choice(int64_t m, int64_t n, int64_t k) { return 1 + daxq::order_by_shape(m, n, k); }

int64_t daxq_linear_splitk_workspace_bytes(int64_t m, int64_t n, int splits) {
    using namespace daxq;
    if (m <= 0 || n <= 0 || splits <= 1) return 0;
    return kCounterBytes + splitk_tiles(m, n) * splits * kPartialBytes;
}

int daxq_linear_w8a8_splitk(int x_fmt, int w_fmt, const void* xq, int64_t ld_xq, const float* sx, const void* wq,
                            int64_t ld_wq, const float* sw, const void* bias, void* out, int64_t ld_out, int64_t m,
                            int64_t n, int64_t k, int splits, void* workspace, int64_t workspace_bytes,
                            daxq_stream_t stream) {
    using namespace daxq;
    bool fp8;
    int f8;
    if (int rc = splitk_formats(x_fmt, w_fmt, fp8, f8)) return rc;
    if (splits < 0 || splits > 64) return fail(DAXQ_ERR_ARG, "linear_splitk: splits must be 0 (library's choice) to 64");
    return fp8 ? launch_gemm_splitk<true>(xq, ld_xq, sx, wq, ld_wq, sw, bias, out, ld_out, m, n, k, splits, workspace,
                                          workspace_bytes, (hipStream_t)stream, f8)
               : launch_gemm_splitk<false>(xq, ld_xq, sx, wq, ld_wq, sw, bias, out, ld_out, m, n, k, splits, workspace,
                                           workspace_bytes, (hipStream_t)stream, 0);
}

int daxq_init(void) {
    using namespace daxq;
    int rc = prepare_tile256_kernels();
    if (!rc) rc = prepare_tile_fp8_kernels();
#define DAXQ_PREP_ALL(FP8, BT, WN)                                        \
    if (!rc) rc = prepare_cfg<FP8, BT, BT, 128, 2, WN, true, 0>();
    DAXQ_PREP_ALL(false, 128, 2)
    DAXQ_PREP_ALL(false, 256, 4)
    DAXQ_PREP_ALL(true, 128, 2)
    DAXQ_PREP_ALL(true, 256, 4)
#undef DAXQ_PREP_ALL
#define DAXQ_PREP_F8(F8)                                                  \
    if (!rc) rc = prepare_cfg<true, 128, 128, 128, 2, 2, true, F8>();      \
    if (!rc) rc = prepare_cfg<true, 256, 256, 128, 2, 4, true, F8>();
    DAXQ_PREP_F8(1)
    DAXQ_PREP_F8(2)
    DAXQ_PREP_F8(3)
#undef DAXQ_PREP_F8
    if (!rc) {  // this device's address of the scratch array behind daxq_linear_w8a8_splitk_static
        void* p = nullptr;
        int dev = 0;
        rc = scratch_of_current_device(&p, &dev);
    }
    return rc;
}

int daxq_linear_w8a8(int x_fmt, int w_fmt, int out_dtype, const void* xq, int64_t ld_xq, const float* sx, const void* wq,
                     int64_t ld_wq, const float* sw, const void* bias, void* out, int64_t ld_out, void* acc,
                     int64_t ld_acc, int64_t m, int64_t n, int64_t k, int kernel, daxq_stream_t stream) {
    using namespace daxq;
    const bool x8 = x_fmt == DAXQ_FMT_E4M3 || x_fmt == DAXQ_FMT_E5M2, w8 = w_fmt == DAXQ_FMT_E4M3 || w_fmt == DAXQ_FMT_E5M2;
    if (x_fmt == DAXQ_FMT_I8 && w_fmt == DAXQ_FMT_I8)
        return launch_gemm<false>(xq, ld_xq, sx, wq, ld_wq, sw, bias, out, ld_out, acc, ld_acc, m, n, k, (hipStream_t)stream, 0,
                                  out_dtype, kernel);
    if (x8 && w8)
        return launch_gemm<true>(xq, ld_xq, sx, wq, ld_wq, sw, bias, out, ld_out, acc, ld_acc, m, n, k, (hipStream_t)stream,
                                 (x_fmt == DAXQ_FMT_E5M2 ? kF8XE5 : 0) | (w_fmt == DAXQ_FMT_E5M2 ? kF8WE5 : 0), out_dtype, kernel);
    return fail(DAXQ_ERR_ARG, "linear: unsupported operand formats x=%d w=%d (int8 x int8, or fp8 x fp8)", x_fmt, w_fmt);
}

// ---- quantiser + GEMM behind one entry point --------------------------------------------------------------------
int daxq_dynamic_linear(int x_dtype, int x_fmt, int w_fmt, int out_dtype, int act_scale_round, const void* x, int64_t ld_x, void* xq,
                        int64_t ld_xq, float* sx, int64_t rows_alloc, const void* wq, int64_t ld_wq, const float* sw,
                        const void* bias, void* out, int64_t ld_out, int64_t m, int64_t n, int64_t k, void* workspace,
                        int64_t workspace_bytes, int kernel, daxq_stream_t stream) {
    using namespace daxq;
    bool fp8;
    int f8;
    if (int rc = splitk_formats(x_fmt, w_fmt, fp8, f8)) return rc;
    if (m < 0 || n < 0 || k <= 0 || rows_alloc < m)
        return fail(DAXQ_ERR_ARG, "dynamic_linear: bad shape m=%lld n=%lld k=%lld rows_alloc=%lld", (long long)m, (long long)n,
                    (long long)k, (long long)rows_alloc);
    const int64_t kp = (k + DAXQ_K_ALIGN - 1) / DAXQ_K_ALIGN * DAXQ_K_ALIGN;
    if (ld_xq < kp || ld_wq < kp)
        return fail(DAXQ_ERR_ARG, "dynamic_linear: ld_xq=%lld and ld_wq=%lld must reach k rounded up to %d (%lld)", (long long)ld_xq,
                    (long long)ld_wq, DAXQ_K_ALIGN, (long long)kp);
    if (m == 0 || n == 0) return DAXQ_OK;
    // the quantiser zero-fills columns [k, kp) of the rows it writes
    const float qmax = x_fmt == DAXQ_FMT_I8 ? 127.0f : x_fmt == DAXQ_FMT_E4M3 ? 448.0f : 57344.0f;
    if (int rc = daxq_act_quant_rows_ex(x, x_dtype, x_fmt, m, k, ld_x, xq, ld_xq, sx, qmax, kEps, act_scale_round, stream)) return rc;
    // Fewer rows than the smallest tile of the tiled kernels: run them on 128 rows of the caller's buffers when those
    // reach that far (the rows beyond m hold whatever the buffers held; an output row depends on its own operand row only).
    const int64_t mg = (m < 128 && rows_alloc >= 128 && n >= 128) ? 128 : m;
    hipStream_t st = (hipStream_t)stream;
    // INT8 launches with few tiles cut K into ranges when the caller brings a workspace (integer partial sums: the
    // same bits as the plain launch); FP8 sums would change with the number of rows, so they stay whole.
    if (!fp8 && workspace && out_dtype == DAXQ_BF16 && kernel == 0) {
        const int splits = splitk_choice(mg, n, kp);
        if (splits > 1 && workspace_bytes >= kCounterBytes + splitk_tiles(mg, n) * splits * kPartialBytes)
            return launch_gemm_splitk<false>(xq, ld_xq, sx, wq, ld_wq, sw, bias, out, ld_out, mg, n, kp, splits, workspace,
                                             workspace_bytes, st, 0);
    }
    return fp8 ? launch_gemm<true>(xq, ld_xq, sx, wq, ld_wq, sw, bias, out, ld_out, nullptr, 0, mg, n, kp, st, f8, out_dtype, kernel)
               : launch_gemm<false>(xq, ld_xq, sx, wq, ld_wq, sw, bias, out, ld_out, nullptr, 0, mg, n, kp, st, 0, out_dtype, kernel);
}

int daxq_dynamic_linear_i8(const void* x, int64_t ld_x, int8_t* xq, int64_t ld_xq, float* sx, const int8_t* wq,
                           int64_t ld_wq, const float* sw, const void* bias, void* out, int64_t ld_out, int64_t m,
                           int64_t n, int64_t k, daxq_stream_t stream) {
    return daxq_dynamic_linear(DAXQ_BF16, DAXQ_FMT_I8, DAXQ_FMT_I8, DAXQ_BF16, DAXQ_SCALE_ROUND_X, x, ld_x, xq, ld_xq, sx, m, wq, ld_wq, sw, bias, out,
                               ld_out, m, n, k, nullptr, 0, 0, stream);
}

int daxq_dynamic_linear_e4m3(const void* x, int64_t ld_x, uint8_t* xq, int64_t ld_xq, float* sx, const uint8_t* wq,
                             int64_t ld_wq, const float* sw, const void* bias, void* out, int64_t ld_out, int64_t m,
                             int64_t n, int64_t k, daxq_stream_t stream) {
    return daxq_dynamic_linear(DAXQ_BF16, DAXQ_FMT_E4M3, DAXQ_FMT_E4M3, DAXQ_BF16, DAXQ_SCALE_ROUND_X, x, ld_x, xq, ld_xq, sx, m, wq, ld_wq, sw, bias,
                               out, ld_out, m, n, k, nullptr, 0, 0, stream);
}

int daxq_dynamic_linear_e5m2_e4m3(const void* x, int64_t ld_x, uint8_t* xq, int64_t ld_xq, float* sx, const uint8_t* wq,
                                  int64_t ld_wq, const float* sw, const void* bias, void* out, int64_t ld_out, int64_t m,
                                  int64_t n, int64_t k, daxq_stream_t stream) {
    return daxq_dynamic_linear(DAXQ_BF16, DAXQ_FMT_E5M2, DAXQ_FMT_E4M3, DAXQ_BF16, DAXQ_SCALE_ROUND_X, x, ld_x, xq, ld_xq, sx, m, wq, ld_wq, sw, bias,
                               out, ld_out, m, n, k, nullptr, 0, 0, stream);
}

int daxq_linear_i8(const int8_t* xq, int64_t ld_xq, const float* sx, const int8_t* wq, int64_t ld_wq, const float* sw,
                   const void* bias, void* out, int64_t ld_out, int32_t* acc, int64_t ld_acc, int64_t m, int64_t n,
                   int64_t k, daxq_stream_t stream) {
    return daxq::launch_gemm<false>(xq, ld_xq, sx, wq, ld_wq, sw, bias, out, ld_out, acc, ld_acc, m, n, k,
                                    (hipStream_t)stream);
}

int daxq_linear_e4m3(const uint8_t* xq, int64_t ld_xq, const float* sx, const uint8_t* wq, int64_t ld_wq,
                     const float* sw, const void* bias, void* out, int64_t ld_out, float* acc, int64_t ld_acc,
                     int64_t m, int64_t n, int64_t k, daxq_stream_t stream) {
    return daxq::launch_gemm<true>(xq, ld_xq, sx, wq, ld_wq, sw, bias, out, ld_out, acc, ld_acc, m, n, k,
                                   (hipStream_t)stream);
}

int daxq_linear_e5m2_e4m3(const uint8_t* xq, int64_t ld_xq, const float* sx, const uint8_t* wq, int64_t ld_wq,
                          const float* sw, const void* bias, void* out, int64_t ld_out, float* acc, int64_t ld_acc,
                          int64_t m, int64_t n, int64_t k, daxq_stream_t stream) {
    return daxq::launch_gemm<true>(xq, ld_xq, sx, wq, ld_wq, sw, bias, out, ld_out, acc, ld_acc, m, n, k,
                                   (hipStream_t)stream, daxq::kF8XE5);
}

}  // extern "C"
