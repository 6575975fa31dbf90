// Device helpers shared by the row quantisers (quant_rows.hip) and the fused producer +
// quantiser kernels (fused_rows.hip): abs-max reduction, the reference's scale rule and the
// leaf quantisers for int8 / OCP e4m3fn / OCP e5m2.
#pragma once

#include "daxq_common.h"

namespace daxq {

typedef unsigned short us2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
    us2 va = __builtin_bit_cast(us2, a), vb = __builtin_bit_cast(us2, b);
    us2 r = __builtin_elementwise_max(va, vb);
    return __builtin_bit_cast(uint32_t, r);
}

// abs-max bits (sign cleared) of a row -> fp32 scale, exactly as the reference rounds it
template <bool ROUND_BF16>
__device__ __forceinline__ float scale_from_amax_bits(uint32_t amax_bits, float qmax) {
    float a = bf16_bits_to_f32(amax_bits);
    float s = a / qmax;  // IEEE binary32 division (hipcc default: correctly rounded)
    if (ROUND_BF16) s = bf16_bits_to_f32(f32_to_bf16_bits(s));
    return fmaxf(s, kEps);
}

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        uint32_t o = (uint32_t)__shfl_xor((int)v, off, 64);
        v = v > o ? v : o;
    }
    return v;
}

__device__ __forceinline__ int q_i8(float x, float inv) {
    float r = rintf(x * inv);  // v_rndne_f32: round half to even
    r = fminf(fmaxf(r, -128.0f), 127.0f);
    return (int)r;
}

// FMT: 0 = int8, 1 = OCP e4m3fn (max 448), 2 = OCP e5m2 (max 57344)
template <int FMT>
__device__ __forceinline__ float q_f8_pre(float x, float s) {
    constexpr float kMax = FMT == 2 ? 57344.0f : 448.0f;
    float v = x / s;  // IEEE division per element
    return fminf(fmaxf(v, -kMax), kMax);
}

template <int FMT>
__device__ __forceinline__ int cvt_pk_f8(float a, float b, int old, bool hi) {
    if constexpr (FMT == 2)
        return hi ? __builtin_amdgcn_cvt_pk_bf8_f32(a, b, old, true) : __builtin_amdgcn_cvt_pk_bf8_f32(a, b, old, false);
    else
        return hi ? __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, true) : __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, false);
}

// 8 bf16 (one 16-byte chunk) -> 8 quantised bytes
template <int FMT>
__device__ __forceinline__ uint2 quant_chunk(const uint4& v, float s, float inv) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t o[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        float f0 = __uint_as_float(w[2 * h] << 16);
        float f1 = __uint_as_float(w[2 * h] & 0xffff0000u);
        float f2 = __uint_as_float(w[2 * h + 1] << 16);
        float f3 = __uint_as_float(w[2 * h + 1] & 0xffff0000u);
        if (FMT != 0) {
            int p = cvt_pk_f8<FMT>(q_f8_pre<FMT>(f0, s), q_f8_pre<FMT>(f1, s), 0, false);
            p = cvt_pk_f8<FMT>(q_f8_pre<FMT>(f2, s), q_f8_pre<FMT>(f3, s), p, true);
            o[h] = (uint32_t)p;
        } else {
            uint32_t b0 = (uint32_t)q_i8(f0, inv) & 0xffu;
            uint32_t b1 = (uint32_t)q_i8(f1, inv) & 0xffu;
            uint32_t b2 = (uint32_t)q_i8(f2, inv) & 0xffu;
            uint32_t b3 = (uint32_t)q_i8(f3, inv) & 0xffu;
            o[h] = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
        }
    }
    return make_uint2(o[0], o[1]);
}

// packed abs-max (two bf16 magnitudes per word) of 8 bf16 values
__device__ __forceinline__ uint32_t chunk_absmax(uint32_t mx, const uint4& v) {
    mx = pk_max_u16(mx, v.x & 0x7fff7fffu);
    mx = pk_max_u16(mx, v.y & 0x7fff7fffu);
    mx = pk_max_u16(mx, v.z & 0x7fff7fffu);
    mx = pk_max_u16(mx, v.w & 0x7fff7fffu);
    return mx;
}

}  // namespace daxq
