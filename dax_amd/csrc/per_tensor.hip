// Per-tensor scales: the scalar-scale variants of the path.
//
// The GEMM and the leaf quantisers take one scale per row / per output channel.  A per-tensor
// scheme (dax/quant/qscheme.py:10-26: the block is the whole tensor) is served by the same kernels
// with the scalar written out as a vector; the three small kernels here produce that scalar and
// its expansion on the device, so that no value travels through the host:
//   * tensor_scale   dynamic per-tensor activation scale from per-row min / max
//                    (dax/quant/nn/dynamic/functional.py:124-129 with a whole-tensor block)
//   * tensor_minmax  running min / max of a calibration observer
//                    (dax/quant/quantization/observer.py:200-214)
//   * broadcast_f32  a stored scalar scale as a vector
//                    (dax/quant/nn/quantized/linear.py:98-100 expands the input scale the same way)
// All are single-workgroup kernels over at most a few hundred thousand values.
#include "quant_rows.h"

namespace daxq {

constexpr int kRedThreads = 1024;

__device__ __forceinline__ void block_minmax(float& lo, float& hi, float* s_lo, float* s_hi) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        lo = min_nan(lo, __shfl_xor(lo, off, 64));
        hi = max_nan(hi, __shfl_xor(hi, off, 64));
    }
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) {
        s_lo[wave] = lo;
        s_hi[wave] = hi;
    }
    __syncthreads();
    lo = s_lo[0];
    hi = s_hi[0];
    for (int w = 1; w < kRedThreads / 64; ++w) {
        lo = min_nan(lo, s_lo[w]);
        hi = max_nan(hi, s_hi[w]);
    }
}

__global__ __launch_bounds__(kRedThreads) void tensor_scale_kernel(const float* __restrict__ mn, const float* __restrict__ mx,
                                                                   int64_t m, float qmax, float eps, int round_bf16,
                                                                   float* __restrict__ scale1, float* __restrict__ expand,
                                                                   int64_t n_expand) {
    __shared__ float s_lo[kRedThreads / 64], s_hi[kRedThreads / 64];
    float lo = __builtin_inff(), hi = -__builtin_inff();
    for (int64_t i = threadIdx.x; i < m; i += kRedThreads) {
        lo = min_nan(lo, mn[i]);
        hi = max_nan(hi, mx[i]);
    }
    block_minmax(lo, hi, s_lo, s_hi);
    const float amax = max_nan(-lo, hi);  // = max |x|: exact, the statistics are the tensor's own values
    float s = amax / qmax;              // IEEE division
    if (round_bf16 == 1) {  // quotient and floor are rounded to the tensor's own element type
        s = round_to_x<DAXQ_BF16>(s);
        eps = round_to_x<DAXQ_BF16>(eps);
    } else if (round_bf16 == 2) {
        s = round_to_x<DAXQ_F16>(s);
        eps = round_to_x<DAXQ_F16>(eps);
    }
    s = max_nan(s, eps);
    if (threadIdx.x == 0) scale1[0] = s;
    for (int64_t i = threadIdx.x; i < n_expand; i += kRedThreads) expand[i] = s;
}

__global__ __launch_bounds__(kRedThreads) void tensor_minmax_kernel(const float* __restrict__ mn, const float* __restrict__ mx,
                                                                    int64_t m, float* __restrict__ min_inout,
                                                                    float* __restrict__ max_inout) {
    __shared__ float s_lo[kRedThreads / 64], s_hi[kRedThreads / 64];
    float lo = __builtin_inff(), hi = -__builtin_inff();
    for (int64_t i = threadIdx.x; i < m; i += kRedThreads) {
        lo = min_nan(lo, mn[i]);
        hi = max_nan(hi, mx[i]);
    }
    block_minmax(lo, hi, s_lo, s_hi);
    if (threadIdx.x == 0) {
        min_inout[0] = min_nan(min_inout[0], lo);
        max_inout[0] = max_nan(max_inout[0], hi);
    }
}

__global__ void broadcast_f32_kernel(const float* __restrict__ src, float* __restrict__ dst, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = src[0];
}

}  // namespace daxq

extern "C" {

int daxq_tensor_scale(const float* row_min, const float* row_max, int64_t m, float qmax, float eps, int round_bf16,
                      float* scale1, float* expand, int64_t n_expand, daxq_stream_t stream) {
    using namespace daxq;
    if (m <= 0 || n_expand < 0 || !(qmax > 0.0f) || !(eps >= 0.0f)) return fail(DAXQ_ERR_ARG, "tensor_scale: bad argument m=%lld n_expand=%lld", (long long)m, (long long)n_expand);
    if (!row_min || !row_max || !scale1 || (n_expand > 0 && !expand)) return fail(DAXQ_ERR_ARG, "tensor_scale: null pointer");
    hipLaunchKernelGGL(tensor_scale_kernel, dim3(1), dim3(kRedThreads), 0, (hipStream_t)stream, row_min, row_max, m, qmax,
                       eps, round_bf16, scale1, expand, n_expand);
    return check_launch("tensor_scale");
}

int daxq_tensor_minmax_update(const float* row_min, const float* row_max, int64_t m, float* min_inout, float* max_inout,
                              daxq_stream_t stream) {
    using namespace daxq;
    if (m <= 0) return fail(DAXQ_ERR_ARG, "tensor_minmax_update: bad argument m=%lld", (long long)m);
    if (!row_min || !row_max || !min_inout || !max_inout) return fail(DAXQ_ERR_ARG, "tensor_minmax_update: null pointer");
    hipLaunchKernelGGL(tensor_minmax_kernel, dim3(1), dim3(kRedThreads), 0, (hipStream_t)stream, row_min, row_max, m,
                       min_inout, max_inout);
    return check_launch("tensor_minmax_update");
}

int daxq_broadcast_f32(const float* src, float* dst, int64_t n, daxq_stream_t stream) {
    using namespace daxq;
    if (n < 0) return fail(DAXQ_ERR_ARG, "broadcast_f32: bad argument");
    if (n == 0) return DAXQ_OK;
    if (!src || !dst) return fail(DAXQ_ERR_ARG, "broadcast_f32: null pointer");
    hipLaunchKernelGGL(broadcast_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, src, dst, n);
    return check_launch("broadcast_f32");
}

}  // extern "C"
