// W8A8 GEMM on gfx950 MFMA with the fused scale / bias / bf16 epilogue.
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
#include "gemm_common.h"

namespace daxq {

// XE5: the activation bytes (MFMA "A" operand here) are e5m2 instead of e4m3fn
template <bool FP8, int BM, int BN, int BK, int WM, int WN, bool DIRECT, bool XE5 = false>
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
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[i], bf[j], acc[i][j], XE5 ? 1 : 0, 0, 0, 0, 0, 0);
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
    //      8*(v/4) + 4*(l/32) + v%4
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const int n = n0 + wn * TN + j * 32 + l31;
        const bool n_ok = n < p.n;
        const int nc = n_ok ? n : p.n - 1;
        const float swv = p.sw[nc];
        const float bv = p.bias ? bf16_bits_to_f32(p.bias[nc]) : 0.0f;
#pragma unroll
        for (int i = 0; i < MB; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = m0 + wm * TM + i * 32 + 8 * (v >> 2) + 4 * hi + (v & 3);
                if (m < p.m && n_ok) {
                    const float sxv = p.sx[m];
                    uint32_t o;
                    if constexpr (!FP8) {
                        float y = (float)acc[i][j][v];  // v_cvt_f32_i32, round to nearest even
                        y = y * sxv;
                        y = y * swv;
                        o = f32_to_bf16_bits(y);
                        if (p.bias) o = f32_to_bf16_bits(bf16_bits_to_f32(o) + bv);
                        if (p.acc) static_cast<int32_t*>(p.acc)[(int64_t)m * p.ldacc + n] = acc[i][j][v];
                    } else {
                        float y = acc[i][j][v] * sxv * swv + bv;
                        o = f32_to_bf16_bits(y);
                        if (p.acc) static_cast<float*>(p.acc)[(int64_t)m * p.ldacc + n] = acc[i][j][v];
                    }
                    p.out[(int64_t)m * p.ldo + n] = (uint16_t)o;
                }
            }
        }
    }
}

static int g_variant = 0;
static int g_gm = 4;

template <bool FP8>
int launch_tile256(const GemmArgs& a, bool x_e5m2, hipStream_t st);
bool tile256_applies(const GemmArgs& a);
template <bool FP8>
int launch_tile256s5(const GemmArgs& a, bool x_e5m2, bool wide, bool small, hipStream_t st);

int prepare_tile256_kernels();

template <bool FP8, int BM, int BN, int BK, int WM, int WN, bool DIRECT, bool XE5 = false>
static int prepare_cfg() {
    static uint64_t lds_set = 0;  // per instantiation
    return ensure_dynamic_lds(reinterpret_cast<const void*>(gemm_w8a8_kernel<FP8, BM, BN, BK, WM, WN, DIRECT, XE5>),
                              2 * (BM + BN) * BK, lds_set);
}

template <bool FP8, int BM, int BN, int BK, int WM, int WN, bool DIRECT, bool XE5 = false>
static int launch_cfg(const GemmArgs& a0, hipStream_t st) {
    GemmArgs a = a0;
    a.tiles_m = (a.m + BM - 1) / BM;
    a.tiles_n = (a.n + BN - 1) / BN;
    constexpr int smem = 2 * (BM + BN) * BK;
    auto kern = gemm_w8a8_kernel<FP8, BM, BN, BK, WM, WN, DIRECT, XE5>;
    if (int rc = prepare_cfg<FP8, BM, BN, BK, WM, WN, DIRECT, XE5>()) return rc;
    const int64_t nt = (int64_t)a.tiles_m * a.tiles_n;
    if (nt > 0x7fffffff) return fail(DAXQ_ERR_ARG, "gemm: too many tiles");
    hipLaunchKernelGGL(kern, dim3((unsigned)nt), dim3(WM * WN * 64), smem, st, a);
    return check_launch("gemm_w8a8");
}

template <bool FP8>
static int launch_gemm(const void* xq, int64_t ld_xq, const float* sx, const void* wq, int64_t ld_wq, const float* sw,
                       const void* bias, void* out, int64_t ld_out, void* acc, int64_t ld_acc, int64_t m, int64_t n,
                       int64_t k, hipStream_t st, bool x_e5m2 = false) {
    if (m < 0 || n < 0 || k <= 0 || ld_xq < k || ld_wq < k || ld_out < n || (acc && ld_acc < n))
        return fail(DAXQ_ERR_ARG, "linear: bad shape m=%lld n=%lld k=%lld", (long long)m, (long long)n, (long long)k);
    if (m == 0 || n == 0) return DAXQ_OK;
    if (!xq || !sx || !wq || !sw || !out) return fail(DAXQ_ERR_ARG, "linear: null pointer");
    if (m > 0x7fffffff || n > 0x7fffffff || k > 0x7fffffff) return fail(DAXQ_ERR_ARG, "linear: dimension exceeds int32");
    if (k % DAXQ_K_ALIGN != 0) return fail(DAXQ_ERR_ALIGN, "linear: k=%lld is not a multiple of %d (zero-pad the operands)", (long long)k, DAXQ_K_ALIGN);
    if (((uintptr_t)xq & 15) || ((uintptr_t)wq & 15) || (ld_xq & 15) || (ld_wq & 15))
        return fail(DAXQ_ERR_ALIGN, "linear: xq/wq must be 16-byte aligned with leading dimensions that are multiples of 16");
    if (((uintptr_t)out & 1) || ((uintptr_t)sx & 3) || ((uintptr_t)sw & 3) || ((uintptr_t)bias & 1) || ((uintptr_t)acc & 3))
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
    a.gm = g_gm;
    switch (g_variant) {
        case 0: {
            // library default: the five-stage kernel on 256x256 tiles once there is one for every second CU, on
            // 128x128 tiles (4x as many workgroups, two per CU) below that, and the generic kernel for operands
            // smaller than one such tile.  Measured at N = K = 5120 (INT8, T-op/s, 128 / 256 tiles):
            // M = 512 -> 1127 / 551, M = 1024 (80 large tiles) -> 1275 / 1055, M = 2048 (160) -> 1542 / 1817;
            // 4096 x 1536 x 1536 (96) -> 1182 / 895, 8192 x 1536 x 1536 (192) -> 1517 / 1587.
            const int64_t tiles256 = ((m + 255) / 256) * ((n + 255) / 256);
            if (tile256_applies(a) && tiles256 >= 128) return launch_tile256s5<FP8>(a, x_e5m2, false, false, st);
            if (m >= 128 && n >= 128 && a.lda < (1 << 26) && a.ldb < (1 << 26)) return launch_tile256s5<FP8>(a, x_e5m2, false, true, st);
            if constexpr (FP8) {
                if (x_e5m2) return launch_cfg<true, 128, 128, 128, 2, 2, true, true>(a, st);
            }
            return launch_cfg<FP8, 128, 128, 128, 2, 2, true>(a, st);
        }
        case 2:
            if (x_e5m2) return fail(DAXQ_ERR_ARG, "linear: gemm variant 2 has no e5m2 form");
            return launch_cfg<FP8, 256, 256, 128, 2, 4, true>(a, st);
        case 5:
            if constexpr (FP8) {
                if (x_e5m2) return launch_cfg<true, 128, 128, 128, 2, 2, true, true>(a, st);
            }
            return launch_cfg<FP8, 128, 128, 128, 2, 2, true>(a, st);
        case 6:
            if (!tile256_applies(a)) return fail(DAXQ_ERR_ARG, "linear: the 256x256 kernel needs m, n >= 256");
            return launch_tile256<FP8>(a, x_e5m2, st);
        case 8:
        case 9:  // 9: INT8 with 32x32x32 MFMAs
            if (!tile256_applies(a)) return fail(DAXQ_ERR_ARG, "linear: the 256x256 kernel needs m, n >= 256");
            return launch_tile256s5<FP8>(a, x_e5m2, g_variant == 9, false, st);
        case 11:  // the five-stage kernel on 128x128 tiles
            if (m < 128 || n < 128 || a.lda >= (1 << 26) || a.ldb >= (1 << 26)) return fail(DAXQ_ERR_ARG, "linear: the 128x128 kernel needs m, n >= 128");
            return launch_tile256s5<FP8>(a, x_e5m2, false, true, st);
        default: return fail(DAXQ_ERR_ARG, "linear: unknown gemm variant %d", g_variant);
    }
}

}  // namespace daxq

extern "C" {

int daxq_init(void) {
    using namespace daxq;
    int rc = prepare_tile256_kernels();
    if (!rc) rc = prepare_cfg<false, 128, 128, 128, 2, 2, true>();
    if (!rc) rc = prepare_cfg<true, 128, 128, 128, 2, 2, true>();
    if (!rc) rc = prepare_cfg<true, 128, 128, 128, 2, 2, true, true>();
    if (!rc) rc = prepare_cfg<false, 256, 256, 128, 2, 4, true>();
    if (!rc) rc = prepare_cfg<true, 256, 256, 128, 2, 4, true>();
    return rc;
}

int daxq_set_gemm_variant(int variant) {
    if (variant >= 1000 && variant < 1064) {  // tuning hook: 1000 + depth of the tile-order groups
        daxq::g_gm = variant - 1000 > 0 ? variant - 1000 : 4;
        return DAXQ_OK;
    }
    if (variant != 0 && variant != 2 && variant != 5 && variant != 6 && variant != 8 && variant != 9 && variant != 11)
        return daxq::fail(DAXQ_ERR_ARG, "unknown gemm variant %d", variant);
    daxq::g_variant = variant;
    return DAXQ_OK;
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
                                   (hipStream_t)stream, true);
}

}  // extern "C"
