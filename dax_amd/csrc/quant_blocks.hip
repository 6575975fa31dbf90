// Block-wise symmetric quantisation for any block shape: the general case of
// dax/quant/nn/dynamic/functional.py:54-148.
//
// The reference views the (contiguous) tensor so that every block becomes a set of whole dimensions
// (_get_reduction_params, :13-51), reduces abs-max over those dimensions, derives one scale per block and
// quantises with the scales broadcast back.  The two kernels here do exactly that for a view of up to 8
// dimensions, each marked reduced or kept:
//   block_scale     one workgroup per block: abs-max over the reduced dimensions -> scale
//   block_quantize  one thread per element: its block's scale -> the leaf quantiser
// The schemes on the hot path never come here: per-token and last-dimension groups are rows of a matrix
// (quant_rows.hip, one pass, the row in registers) and per-tensor has its own reduction (per_tensor.hip).
// These kernels serve what is left -- per-channel activations, 2-d tiles, blocks over leading dimensions --
// with plain strided accesses, and any of the three element types.
#include "quant_rows.h"

namespace daxq {

constexpr int kMaxDims = 8;

struct BlockView {
    int nd;
    int64_t size[kMaxDims];
    int64_t stride[kMaxDims];  // in elements, of the contiguous view
    int reduced[kMaxDims];
};

template <int XT>
struct XW {
    typedef uint16_t type;
};
template <>
struct XW<DAXQ_F32> {
    typedef uint32_t type;
};

// offset of the element with mixed-radix index `idx` over the dimensions whose reduced flag equals `which`
__device__ __forceinline__ int64_t offset_of(const BlockView& v, int64_t idx, int which) {
    int64_t off = 0;
    for (int d = v.nd - 1; d >= 0; --d) {
        if (v.reduced[d] != which) continue;
        const int64_t c = idx % v.size[d];
        idx /= v.size[d];
        off += c * v.stride[d];
    }
    return off;
}

template <int XT, bool ROUND>
__global__ __launch_bounds__(256) void block_scale_kernel(const void* __restrict__ xv, const BlockView v, int64_t n_red,
                                                          float qmax, float eps, float* __restrict__ scale) {
    typedef typename XW<XT>::type word_t;
    constexpr uint32_t kAbs = XT == DAXQ_F32 ? 0x7fffffffu : 0x7fffu;
    __shared__ uint32_t red[4];
    const word_t* x = static_cast<const word_t*>(xv) + offset_of(v, blockIdx.x, 0);
    uint32_t mx = 0;
    for (int64_t r = threadIdx.x; r < n_red; r += 256) {
        const uint32_t a = x[offset_of(v, r, 1)] & kAbs;
        mx = a > mx ? a : mx;
    }
    mx = wave_max_u32(mx);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t amax = red[0];
        amax = red[1] > amax ? red[1] : amax;
        amax = red[2] > amax ? red[2] : amax;
        amax = red[3] > amax ? red[3] : amax;
        scale[blockIdx.x] = scale_from_amax_bits_rt<XT>(amax, qmax, eps, ROUND ? 1 : 0);
    }
}

// f32 rounded to the arithmetic type CT of the leaf quantiser (DAXQ_F32: no rounding)
__device__ __forceinline__ float round_ct(float v, int ct) {
    if (ct == DAXQ_BF16) return round_to_x<DAXQ_BF16>(v);
    if (ct == DAXQ_F16) return round_to_x<DAXQ_F16>(v);
    return v;
}

// st / ct: the element type of the scale the caller asked for, and the type torch's type promotion makes of (x, scale).
// The reference's wrappers always ask for an fp32 scale, and then everything below is fp32.  With a scale of a 16-bit
// type (dax/quant/nn/dynamic/functional.py:128-129) the leaf quantisers (dax/quant/nn/quantized/functional.py:11-20)
// round 1.0 / scale to the scale's type, and x * inv and x / scale to the promoted type: bf16 x with a bf16 scale
// computes in bf16, bf16 x with an fp16 scale in fp32 (but with the reciprocal rounded to fp16).
template <int XT, int FMT>
__global__ __launch_bounds__(256) void block_quantize_kernel(const void* __restrict__ xv, const BlockView v, int64_t total,
                                                             const float* __restrict__ scale, uint8_t* __restrict__ q, int st, int ct) {
    typedef typename XW<XT>::type word_t;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    // index of the element's block among the kept dimensions (row-major), from its coordinates in the view
    int64_t rest = i, blk = 0, mul = 1;
    for (int d = v.nd - 1; d >= 0; --d) {
        const int64_t c = rest % v.size[d];
        rest /= v.size[d];
        if (!v.reduced[d]) {
            blk += c * mul;
            mul *= v.size[d];
        }
    }
    const float s = scale[blk];
    const float f = x_bits_to_f32<XT>(static_cast<const word_t*>(xv)[i]);
    if constexpr (FMT == 0) {
        if (ct == DAXQ_F32 && st == DAXQ_F32) {
            q[i] = (uint8_t)(q_i8_bits(f, 1.0f / s) & 0xffu);
        } else {
            const float inv = round_ct(1.0f / s, st);
            float r = round_ct(f * inv, ct);  // (the product of two 16-bit floats is exact in fp32: one rounding)
            r = rintf(r);                     // an integer below 2^8 (bf16) or 2^11 (fp16) in magnitude is exact in that type; larger ones clamp
            r = min_nan(max_nan(r, -128.0f), 127.0f);
            q[i] = (uint8_t)(int8_t)(r != r ? 0.0f : r);
        }
    } else {
        if (ct == DAXQ_F32) {
            q[i] = (uint8_t)(cvt_pk_f8<FMT>(q_f8_pre<FMT, true>(f, s, 0.0f), 0.0f, 0, false) & 0xff);
        } else {
            constexpr float kMax = FMT == 2 ? 57344.0f : 448.0f;
            float r = round_ct(f / s, ct);
            r = min_nan(max_nan(r, -kMax), kMax);
            q[i] = (uint8_t)(cvt_pk_f8<FMT>(r, 0.0f, 0, false) & 0xff);
        }
    }
}

// fills in the view from host arrays; returns the element count, or -1 on a bad argument
static int64_t make_view(BlockView& v, int nd, const int64_t* view_shape, const int32_t* reduced, int64_t& n_kept, int64_t& n_red) {
    if (nd <= 0 || nd > kMaxDims || !view_shape || !reduced) return -1;
    v.nd = nd;
    int64_t total = 1;
    n_kept = n_red = 1;
    for (int d = nd - 1; d >= 0; --d) {
        if (view_shape[d] <= 0) return view_shape[d] == 0 ? 0 : -1;
        v.size[d] = view_shape[d];
        v.stride[d] = total;
        v.reduced[d] = reduced[d] ? 1 : 0;
        total *= view_shape[d];
        (reduced[d] ? n_red : n_kept) *= view_shape[d];
    }
    for (int d = nd; d < kMaxDims; ++d) {
        v.size[d] = 1;
        v.stride[d] = 0;
        v.reduced[d] = 0;
    }
    return total;
}

}  // namespace daxq

extern "C" {

int daxq_block_scale(const void* x, int x_dtype, int nd, const int64_t* view_shape, const int32_t* reduced, float qmax,
                     float eps, int round_to_x, float* scale, daxq_stream_t stream) {
    using namespace daxq;
    BlockView v;
    int64_t n_kept, n_red;
    const int64_t total = make_view(v, nd, view_shape, reduced, n_kept, n_red);
    if (total < 0 || !(qmax > 0.0f) || !(eps >= 0.0f)) return fail(DAXQ_ERR_ARG, "block_scale: bad view (1 to %d positive dimensions), quant_max or eps", kMaxDims);
    if (total == 0) return DAXQ_OK;
    if (!x || !scale) return fail(DAXQ_ERR_ARG, "block_scale: null pointer");
    if (n_kept > 0x7fffffff) return fail(DAXQ_ERR_ARG, "block_scale: too many blocks");
    const dim3 grid((unsigned)n_kept), block(256);
    hipStream_t st = (hipStream_t)stream;
#define DAXQ_BS(XT)                                                                                             \
    if (round_to_x) hipLaunchKernelGGL((block_scale_kernel<XT, true>), grid, block, 0, st, x, v, n_red, qmax, eps, scale); \
    else hipLaunchKernelGGL((block_scale_kernel<XT, false>), grid, block, 0, st, x, v, n_red, qmax, eps, scale)
    switch (x_dtype) {
        case DAXQ_BF16: DAXQ_BS(DAXQ_BF16); break;
        case DAXQ_F16: DAXQ_BS(DAXQ_F16); break;
        case DAXQ_F32: DAXQ_BS(DAXQ_F32); break;
        default: return fail(DAXQ_ERR_ARG, "block_scale: unknown element type %d", x_dtype);
    }
#undef DAXQ_BS
    return check_launch("block_scale");
}

int daxq_block_quantize(const void* x, int x_dtype, int q_fmt, int nd, const int64_t* view_shape, const int32_t* reduced,
                        const float* scale, int scale_dtype, void* q, daxq_stream_t stream) {
    using namespace daxq;
    BlockView v;
    int64_t n_kept, n_red;
    const int64_t total = make_view(v, nd, view_shape, reduced, n_kept, n_red);
    if (total < 0) return fail(DAXQ_ERR_ARG, "block_quantize: bad view (1 to %d positive dimensions)", kMaxDims);
    if (total == 0) return DAXQ_OK;
    if (!x || !scale || !q) return fail(DAXQ_ERR_ARG, "block_quantize: null pointer");
    if (scale_dtype != DAXQ_F32 && scale_dtype != DAXQ_BF16 && scale_dtype != DAXQ_F16)
        return fail(DAXQ_ERR_ARG, "block_quantize: unknown scale type %d", scale_dtype);
    // type promotion of (x, scale): the same 16-bit type on both sides stays, anything else is fp32
    const int sk = scale_dtype, ct = (x_dtype == scale_dtype) ? x_dtype : DAXQ_F32;
    if ((total + 255) / 256 > 0x7fffffff) return fail(DAXQ_ERR_ARG, "block_quantize: tensor too large");
    const dim3 grid((unsigned)((total + 255) / 256)), block(256);
    hipStream_t st = (hipStream_t)stream;
    uint8_t* qp = static_cast<uint8_t*>(q);
#define DAXQ_BQ(XT)                                                                                                   \
    switch (q_fmt) {                                                                                                  \
        case DAXQ_FMT_I8: hipLaunchKernelGGL((block_quantize_kernel<XT, 0>), grid, block, 0, st, x, v, total, scale, qp, sk, ct); break;   \
        case DAXQ_FMT_E4M3: hipLaunchKernelGGL((block_quantize_kernel<XT, 1>), grid, block, 0, st, x, v, total, scale, qp, sk, ct); break; \
        case DAXQ_FMT_E5M2: hipLaunchKernelGGL((block_quantize_kernel<XT, 2>), grid, block, 0, st, x, v, total, scale, qp, sk, ct); break; \
        default: return fail(DAXQ_ERR_ARG, "block_quantize: unknown quantised format %d", q_fmt);                    \
    }
    switch (x_dtype) {
        case DAXQ_BF16: DAXQ_BQ(DAXQ_BF16) break;
        case DAXQ_F16: DAXQ_BQ(DAXQ_F16) break;
        case DAXQ_F32: DAXQ_BQ(DAXQ_F32) break;
        default: return fail(DAXQ_ERR_ARG, "block_quantize: unknown element type %d", x_dtype);
    }
#undef DAXQ_BQ
    return check_launch("block_quantize");
}

}  // extern "C"
