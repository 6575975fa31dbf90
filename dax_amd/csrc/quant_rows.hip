// Row-wise symmetric quantisation of a bf16 / fp16 / fp32 matrix to int8, OCP e4m3fn or OCP e5m2.
//
// One launch covers both uses on the path:
//   * dynamic per-token activation quantisation (scale rounded to bf16 first, as
//     the eager dtype chain of dax/quant/nn/dynamic/functional.py:124-129 does), and
//   * one-time per-output-channel weight quantisation (scale kept in fp32,
//     dax/quant/quantization/observer.py:97-134).
// The element rule is the leaf quantiser of dax/quant/nn/quantized/functional.py:11-20:
//   int8:  clamp(rint(f32(x) * (1.0f / s)), -128, 127)      reciprocal-multiply
//   e4m3:  e4m3fn_rne(clamp(f32(x) / s, -448, 448))         true division
//   e5m2:  e5m2_rne(clamp(f32(x) / s, -57344, 57344))       true division (activations only)
//
// HBM-bound: 2 B read + 1 B written per element.  The fast kernel gives one
// 64-lane wavefront a whole row, keeps the row in VGPRs between the abs-max pass
// and the quantise pass (so HBM is read once), reduces the abs-max with packed
// u16 max + wavefront shuffles, and writes 8 quantised bytes per lane per store.
#include "quant_rows.h"

namespace daxq {

// Fast path: one wavefront per row, the row lives in registers.
// Requires k % 8 == 0, ld_x % 8 == 0, ld_q % 8 == 0, 16-byte aligned x, 8-byte aligned q,
// and kfill / 8 <= NCH * 64.
// SCALE_IN: the per-row scale is an input (leaf quantiser) instead of being derived from the row.
// XT: element type of x, DAXQ_BF16 or DAXQ_F16 (8 elements per 16-byte chunk either way).
template <int NCH, int FMT, bool ROUND_BF16, bool SCALE_IN, int XT = DAXQ_BF16>
__global__ __launch_bounds__(256) void quant_rows_wave(const uint16_t* __restrict__ x, int64_t m, int k,
                                                       int64_t ld_x, uint8_t* __restrict__ q, int64_t ld_q, int kfill,
                                                       float* __restrict__ scale, float qmax, float eps, int round_x) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= m) return;
    const uint4* xr = reinterpret_cast<const uint4*>(x + row * ld_x);
    const int nch = k >> 3;
    const int npad = kfill >> 3;  // columns [k, kfill) are written as zeros

    uint4 v[NCH];
    uint32_t mx = 0;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int c = i * 64 + lane;
        if (c < nch) {
            v[i] = load_stream_16(xr + c);
        } else {
            v[i] = make_uint4(0, 0, 0, 0);
        }
    }
    float s;
    if constexpr (SCALE_IN) {
        s = scale[row];
    } else {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            mx = pk_max_u16(mx, v[i].x & 0x7fff7fffu);
            mx = pk_max_u16(mx, v[i].y & 0x7fff7fffu);
            mx = pk_max_u16(mx, v[i].z & 0x7fff7fffu);
            mx = pk_max_u16(mx, v[i].w & 0x7fff7fffu);
        }
        uint32_t amax = (mx & 0xffffu) > (mx >> 16) ? (mx & 0xffffu) : (mx >> 16);
        amax = wave_max_u32(amax);
        s = scale_from_amax_bits_rt<XT>(amax, qmax, eps, round_x);
        if (lane == 0) scale[row] = s;
    }
    const float inv = 1.0f / s;  // IEEE division, not v_rcp_f32

    uint2* qr = reinterpret_cast<uint2*>(q + row * ld_q);
    // Two forms of the store loop.  The fast one, for a bf16 row quantised with its own scale at no more than the
    // format's maximum: no clamp (dead code there, quant_rows.h), and for FP8 the reciprocal sequence, which is verified
    // exhaustively for bf16 elements under bf16-rounded scales.  The general one -- fp16 rows, a scale from the caller,
    // a quant_max beyond the format's maximum, an FP8 row whose scale stays in fp32 -- divides and clamps.  The choice
    // is uniform over the launch.
    constexpr float kFmtMax = FMT == 0 ? 127.0f : FMT == 1 ? 448.0f : 57344.0f;
    constexpr bool kFastForm = !SCALE_IN && XT == DAXQ_BF16;
    if (kFastForm && qmax <= kFmtMax && (FMT == 0 || round_x)) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int c = i * 64 + lane;
            if (c < nch) store_stream_8(qr + c, quant_chunk<FMT, false, XT, false>(v[i], s, inv));
            else if (c < npad) store_stream_8(qr + c, make_uint2(0, 0));
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int c = i * 64 + lane;
        if (c < nch) {
            store_stream_8(qr + c, quant_chunk<FMT, (FMT != 0), XT>(v[i], s, inv));
        } else if (c < npad) {
            store_stream_8(qr + c, make_uint2(0, 0));
        }
    }
}

// General path: any k / alignment / row length / element type; one 256-thread block per row, two passes.
template <int XT>
struct XWord {
    typedef uint16_t type;
};
template <>
struct XWord<DAXQ_F32> {
    typedef uint32_t type;
};

template <int FMT, bool ROUND_BF16, bool SCALE_IN, int XT = DAXQ_BF16>
__global__ __launch_bounds__(256) void quant_rows_block(const void* __restrict__ xv, int64_t m, int64_t k,
                                                        int64_t ld_x, uint8_t* __restrict__ q, int64_t ld_q, int64_t kfill,
                                                        float* __restrict__ scale, float qmax, float eps, int round_x) {
    typedef typename XWord<XT>::type word_t;
    constexpr uint32_t kAbs = XT == DAXQ_F32 ? 0x7fffffffu : 0x7fffu;
    __shared__ uint32_t red[4];
    const int64_t row = blockIdx.x;
    const word_t* xr = static_cast<const word_t*>(xv) + row * ld_x;
    float s;
    if constexpr (SCALE_IN) {
        s = scale[row];
    } else {
        uint32_t mx = 0;
        for (int64_t c = threadIdx.x; c < k; c += 256) {
            uint32_t a = xr[c] & kAbs;
            mx = a > mx ? a : mx;
        }
        mx = wave_max_u32(mx);
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
        __syncthreads();
        uint32_t amax = red[0];
        amax = red[1] > amax ? red[1] : amax;
        amax = red[2] > amax ? red[2] : amax;
        amax = red[3] > amax ? red[3] : amax;
        s = scale_from_amax_bits_rt<XT>(amax, qmax, eps, round_x);
        if (threadIdx.x == 0) scale[row] = s;
    }
    const float inv = 1.0f / s;
    uint8_t* qr = q + row * ld_q;
    for (int64_t c = threadIdx.x; c < kfill; c += 256) {
        uint8_t o = 0;
        if (c < k) {
            float f = x_bits_to_f32<XT>(xr[c]);
            if (FMT != 0) {
                // the reciprocal sequence is verified exhaustively for bf16 elements only; other types divide
                const float pre = (SCALE_IN || XT != DAXQ_BF16 || round_x) ? q_f8_pre<FMT, SCALE_IN || XT != DAXQ_BF16>(f, s, inv)
                                                                           : q_f8_pre<FMT, true>(f, s, inv);
                o = (uint8_t)(cvt_pk_f8<FMT>(pre, 0.0f, 0, false) & 0xff);
            } else {
                o = (uint8_t)(q_i8_bits(f, inv) & 0xffu);
            }
        }
        qr[c] = o;
    }
}

template <int FMT, bool ROUND_BF16, bool SCALE_IN, int XT>
static int launch_quant_rows_t(const void* x, int64_t m, int64_t k, int64_t ld_x, void* q, int64_t ld_q, float* scale,
                               float qmax, hipStream_t st, float eps, int round_x) {
    constexpr int XB = XT == DAXQ_F32 ? 4 : 2;
    if (m < 0 || k <= 0 || ld_x < k || ld_q < k) return fail(DAXQ_ERR_ARG, "quant_rows: bad shape m=%lld k=%lld ld_x=%lld ld_q=%lld",
                                                               (long long)m, (long long)k, (long long)ld_x, (long long)ld_q);
    if (m == 0) return DAXQ_OK;
    if (!x || !q || !scale) return fail(DAXQ_ERR_ARG, "quant_rows: null pointer");
    const int64_t kfill = fill_width(k, ld_q);
    if (((uintptr_t)x & (XB - 1)) != 0 || ((uintptr_t)scale & 3) != 0) return fail(DAXQ_ERR_ALIGN, "quant_rows: x must be element aligned and scale 4-byte aligned");
    uint8_t* qp = static_cast<uint8_t*>(q);
    if constexpr (XT != DAXQ_F32) {
        const uint16_t* xp = static_cast<const uint16_t*>(x);
        const bool vec_ok = (k % 8 == 0) && (ld_x % 8 == 0) && (ld_q % 8 == 0) && (((uintptr_t)x & 15) == 0) &&
                            (((uintptr_t)q & 7) == 0) && (kfill / 8 <= 36 * 64) && (m <= (int64_t)4 * 0x7fffffff);
        if (vec_ok) {
            const int nchunks = (int)((kfill / 8 + 63) / 64);
            const dim3 grid((unsigned)((m + 3) / 4)), block(256);
#define DAXQ_Q_CASE(N)                                                                                      \
    if (nchunks <= N) {                                                                                     \
        hipLaunchKernelGGL((quant_rows_wave<N, FMT, ROUND_BF16, SCALE_IN, XT>), grid, block, 0, st, xp, m, (int)k, ld_x, qp, \
                           ld_q, (int)kfill, scale, qmax, eps, round_x);                                              \
        return check_launch("quant_rows_wave");                                                             \
    }
            DAXQ_Q_CASE(2)
            DAXQ_Q_CASE(4)
            DAXQ_Q_CASE(8)
            DAXQ_Q_CASE(12)
            DAXQ_Q_CASE(20)
            DAXQ_Q_CASE(28)
            DAXQ_Q_CASE(36)
#undef DAXQ_Q_CASE
        }
    }
    if (m > 0x7fffffff) return fail(DAXQ_ERR_ARG, "quant_rows: too many rows for the general kernel");
    hipLaunchKernelGGL((quant_rows_block<FMT, ROUND_BF16, SCALE_IN, XT>), dim3((unsigned)m), dim3(256), 0, st, x, m, k, ld_x, qp,
                       ld_q, kfill, scale, qmax, eps, round_x);
    return check_launch("quant_rows_block");
}

// eps, round_x: floor and rounding of a dynamic scale (scale_from_amax_bits_rt); unused when the scale is an input
template <int FMT, bool ROUND_BF16, bool SCALE_IN>
static int launch_quant_rows(const void* x, int64_t m, int64_t k, int64_t ld_x, void* q, int64_t ld_q, float* scale,
                             float qmax, hipStream_t st, int x_dtype = DAXQ_BF16, float eps = kEps, int round_x = 1) {
    if (!SCALE_IN && (!(qmax > 0.0f) || !(eps >= 0.0f))) return fail(DAXQ_ERR_ARG, "quant_rows: quant_max must be positive and eps not negative");
    switch (x_dtype) {
        case DAXQ_BF16: return launch_quant_rows_t<FMT, ROUND_BF16, SCALE_IN, DAXQ_BF16>(x, m, k, ld_x, q, ld_q, scale, qmax, st, eps, round_x);
        case DAXQ_F16: return launch_quant_rows_t<FMT, ROUND_BF16, SCALE_IN, DAXQ_F16>(x, m, k, ld_x, q, ld_q, scale, qmax, st, eps, round_x);
        case DAXQ_F32: return launch_quant_rows_t<FMT, ROUND_BF16, SCALE_IN, DAXQ_F32>(x, m, k, ld_x, q, ld_q, scale, qmax, st, eps, round_x);
        default: return fail(DAXQ_ERR_ARG, "quant_rows: unknown element type %d", x_dtype);
    }
}

// qmax <= 0: the format's own maximum
template <bool ROUND_BF16, bool SCALE_IN>
static int launch_quant_rows_fmt(int q_fmt, const void* x, int x_dtype, int64_t m, int64_t k, int64_t ld_x, void* q,
                                 int64_t ld_q, float* scale, hipStream_t st, float qmax = 0.0f, float eps = kEps, int round_x = 1) {
    switch (q_fmt) {
        case DAXQ_FMT_I8: return launch_quant_rows<0, ROUND_BF16, SCALE_IN>(x, m, k, ld_x, q, ld_q, scale, qmax > 0.0f ? qmax : 127.0f, st, x_dtype, eps, round_x);
        case DAXQ_FMT_E4M3: return launch_quant_rows<1, ROUND_BF16, SCALE_IN>(x, m, k, ld_x, q, ld_q, scale, qmax > 0.0f ? qmax : 448.0f, st, x_dtype, eps, round_x);
        case DAXQ_FMT_E5M2: return launch_quant_rows<2, ROUND_BF16, SCALE_IN>(x, m, k, ld_x, q, ld_q, scale, qmax > 0.0f ? qmax : 57344.0f, st, x_dtype, eps, round_x);
        default: return fail(DAXQ_ERR_ARG, "quant_rows: unknown quantised format %d", q_fmt);
    }
}


// Per-row min and max of a bf16 / fp16 / fp32 matrix in fp32 (weight observer statistics).
template <int XT>
__global__ __launch_bounds__(256) void row_minmax_kernel(const void* __restrict__ xv, int64_t k, int64_t ld_x,
                                                         float* __restrict__ mn, float* __restrict__ mx) {
    typedef typename XWord<XT>::type word_t;
    __shared__ float rlo[4], rhi[4];
    const int64_t row = blockIdx.x;
    const word_t* xr = static_cast<const word_t*>(xv) + row * ld_x;
    float lo = __builtin_inff(), hi = -__builtin_inff();
    for (int64_t c = threadIdx.x; c < k; c += 256) {
        float f = x_bits_to_f32<XT>(xr[c]);
        lo = min_nan(lo, f);
        hi = max_nan(hi, f);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        lo = min_nan(lo, __shfl_xor(lo, off, 64));
        hi = max_nan(hi, __shfl_xor(hi, off, 64));
    }
    if ((threadIdx.x & 63) == 0) {
        rlo[threadIdx.x >> 6] = lo;
        rhi[threadIdx.x >> 6] = hi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        mn[row] = min_nan(min_nan(rlo[0], rlo[1]), min_nan(rlo[2], rlo[3]));
        mx[row] = max_nan(max_nan(rhi[0], rhi[1]), max_nan(rhi[2], rhi[3]));
    }
}

// scale[i] = max( max(-min[i], max[i]) / qmax, eps ), all in fp32
__global__ void scale_from_minmax_kernel(const float* __restrict__ mn, const float* __restrict__ mx, int64_t n,
                                         float qmax, float eps, float* __restrict__ scale) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const float a = max_nan(-mn[i], mx[i]);
        scale[i] = max_nan(a / qmax, eps);
    }
}

}  // namespace daxq

extern "C" {

int daxq_act_quant_i8(const void* x, int64_t m, int64_t k, int64_t ld_x, int8_t* q, int64_t ld_q, float* scale,
                      daxq_stream_t stream) {
    return daxq::launch_quant_rows<0, true, false>(x, m, k, ld_x, q, ld_q, scale, 127.0f, (hipStream_t)stream);
}

int daxq_act_quant_e4m3(const void* x, int64_t m, int64_t k, int64_t ld_x, uint8_t* q, int64_t ld_q, float* scale,
                        daxq_stream_t stream) {
    return daxq::launch_quant_rows<1, true, false>(x, m, k, ld_x, q, ld_q, scale, 448.0f, (hipStream_t)stream);
}

int daxq_act_quant_e5m2(const void* x, int64_t m, int64_t k, int64_t ld_x, uint8_t* q, int64_t ld_q, float* scale,
                        daxq_stream_t stream) {
    return daxq::launch_quant_rows<2, true, false>(x, m, k, ld_x, q, ld_q, scale, 57344.0f, (hipStream_t)stream);
}

int daxq_quantize_rows_i8(const void* x, int64_t m, int64_t k, int64_t ld_x, const float* scale, int8_t* q,
                          int64_t ld_q, daxq_stream_t stream) {
    return daxq::launch_quant_rows<0, false, true>(x, m, k, ld_x, q, ld_q, const_cast<float*>(scale), 127.0f,
                                                       (hipStream_t)stream);
}

int daxq_quantize_rows_e4m3(const void* x, int64_t m, int64_t k, int64_t ld_x, const float* scale, uint8_t* q,
                            int64_t ld_q, daxq_stream_t stream) {
    return daxq::launch_quant_rows<1, false, true>(x, m, k, ld_x, q, ld_q, const_cast<float*>(scale), 448.0f,
                                                      (hipStream_t)stream);
}

int daxq_quantize_rows_e5m2(const void* x, int64_t m, int64_t k, int64_t ld_x, const float* scale, uint8_t* q,
                            int64_t ld_q, daxq_stream_t stream) {
    return daxq::launch_quant_rows<2, false, true>(x, m, k, ld_x, q, ld_q, const_cast<float*>(scale), 57344.0f,
                                                      (hipStream_t)stream);
}

int daxq_row_minmax_t(const void* x, int x_dtype, int64_t m, int64_t k, int64_t ld_x, float* min_out, float* max_out,
                      daxq_stream_t stream) {
    using namespace daxq;
    if (m < 0 || k <= 0 || ld_x < k || m > 0x7fffffff) return fail(DAXQ_ERR_ARG, "row_minmax: bad shape m=%lld k=%lld", (long long)m, (long long)k);
    if (m == 0) return DAXQ_OK;
    if (!x || !min_out || !max_out) return fail(DAXQ_ERR_ARG, "row_minmax: null pointer");
    const dim3 grid((unsigned)m), block(256);
    switch (x_dtype) {
        case DAXQ_BF16: hipLaunchKernelGGL(row_minmax_kernel<DAXQ_BF16>, grid, block, 0, (hipStream_t)stream, x, k, ld_x, min_out, max_out); break;
        case DAXQ_F16: hipLaunchKernelGGL(row_minmax_kernel<DAXQ_F16>, grid, block, 0, (hipStream_t)stream, x, k, ld_x, min_out, max_out); break;
        case DAXQ_F32: hipLaunchKernelGGL(row_minmax_kernel<DAXQ_F32>, grid, block, 0, (hipStream_t)stream, x, k, ld_x, min_out, max_out); break;
        default: return fail(DAXQ_ERR_ARG, "row_minmax: unknown element type %d", x_dtype);
    }
    return check_launch("row_minmax");
}

int daxq_row_minmax(const void* x, int64_t m, int64_t k, int64_t ld_x, float* min_out, float* max_out,
                    daxq_stream_t stream) {
    return daxq_row_minmax_t(x, DAXQ_BF16, m, k, ld_x, min_out, max_out, stream);
}

int daxq_act_quant_rows(const void* x, int x_dtype, int q_fmt, int64_t m, int64_t k, int64_t ld_x, void* q, int64_t ld_q,
                        float* scale, daxq_stream_t stream) {
    return daxq::launch_quant_rows_fmt<true, false>(q_fmt, x, x_dtype, m, k, ld_x, q, ld_q, scale, (hipStream_t)stream);
}

int daxq_act_quant_rows_ex(const void* x, int x_dtype, int q_fmt, int64_t m, int64_t k, int64_t ld_x, void* q, int64_t ld_q,
                           float* scale, float quant_max, float eps, int scale_round, daxq_stream_t stream) {
    if (scale_round != DAXQ_SCALE_ROUND_X && scale_round != DAXQ_SCALE_ROUND_NONE)
        return daxq::fail(DAXQ_ERR_ARG, "act_quant_rows_ex: unknown scale rounding %d", scale_round);
    if (!(quant_max > 0.0f)) return daxq::fail(DAXQ_ERR_ARG, "act_quant_rows_ex: quant_max must be positive");
    return daxq::launch_quant_rows_fmt<true, false>(q_fmt, x, x_dtype, m, k, ld_x, q, ld_q, scale, (hipStream_t)stream, quant_max,
                                                    eps, scale_round == DAXQ_SCALE_ROUND_X);
}

int daxq_quantize_rows(const void* x, int x_dtype, int q_fmt, int64_t m, int64_t k, int64_t ld_x, const float* scale,
                       void* q, int64_t ld_q, daxq_stream_t stream) {
    return daxq::launch_quant_rows_fmt<false, true>(q_fmt, x, x_dtype, m, k, ld_x, q, ld_q, const_cast<float*>(scale),
                                                    (hipStream_t)stream);
}

int daxq_scale_from_minmax(const float* min_in, const float* max_in, int64_t n, float qmax, float* scale,
                           daxq_stream_t stream) {
    return daxq_scale_from_minmax_eps(min_in, max_in, n, qmax, daxq::kEps, scale, stream);
}

int daxq_scale_from_minmax_eps(const float* min_in, const float* max_in, int64_t n, float qmax, float eps, float* scale,
                               daxq_stream_t stream) {
    using namespace daxq;
    if (n < 0 || !(qmax > 0.0f) || eps != eps) return fail(DAXQ_ERR_ARG, "scale_from_minmax: bad argument");
    if (n == 0) return DAXQ_OK;
    if (!min_in || !max_in || !scale) return fail(DAXQ_ERR_ARG, "scale_from_minmax: null pointer");
    hipLaunchKernelGGL(scale_from_minmax_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       min_in, max_in, n, qmax, eps, scale);
    return check_launch("scale_from_minmax");
}

}  // extern "C"
