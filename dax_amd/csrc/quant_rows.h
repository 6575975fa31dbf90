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

// Element type of the tensor being quantised: XT = DAXQ_BF16 / DAXQ_F16 (two per 32-bit word) / DAXQ_F32.
// The bit pattern of a non-negative value orders like the value in all three, NaN above infinity.
template <int XT>
__device__ __forceinline__ float x_bits_to_f32(uint32_t b) {
    if constexpr (XT == DAXQ_BF16) return __uint_as_float(b << 16);
    else if constexpr (XT == DAXQ_F16) return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
    else return __uint_as_float(b);
}

// f32 rounded to the element type (round to nearest even, subnormals of fp16 included), as a float
template <int XT>
__device__ __forceinline__ float round_to_x(float s) {
    if constexpr (XT == DAXQ_BF16) {
        if (s != s) return s;
        return bf16_bits_to_f32(f32_to_bf16_bits(s));
    } else if constexpr (XT == DAXQ_F16) {
        asm volatile("" : "+v"(s));  // keeps the conversion a conversion (no fold with the operation that produced s)
        return (float)(_Float16)s;
    } else {
        return s;
    }
}

// Columns [k, fill_width) of a quantised row are written as zeros: up to the next multiple of the GEMM's K granularity,
// as far as the row reaches.  A row stride beyond that (rows kept apart on purpose, or a column slice of a wider
// buffer) is left alone.
inline int64_t fill_width(int64_t k, int64_t ld_q) {
    const int64_t kp = (k + DAXQ_K_ALIGN - 1) / DAXQ_K_ALIGN * DAXQ_K_ALIGN;
    return kp < ld_q ? kp : ld_q;
}

// abs-max bits (sign cleared) of a block -> fp32 scale, exactly as the reference rounds it: the quotient is
// computed and floored in the tensor's own dtype when ROUND (dynamic activations,
// dax/quant/nn/dynamic/functional.py:124-129), in fp32 otherwise (weight observer).
template <bool ROUND, int XT = DAXQ_BF16>
__device__ __forceinline__ float scale_from_amax_bits(uint32_t amax_bits, float qmax) {
    float a = x_bits_to_f32<XT>(amax_bits);
    float s = a / qmax;  // IEEE binary32 division (hipcc default: correctly rounded)
    if (ROUND) s = round_to_x<XT>(s);
    return max_nan(s, kEps);  // clamp(min=eps): a NaN abs-max (a NaN anywhere in the row) stays NaN
}

// The same rule with the caller's floor and the rounding chosen at run time (uniform over the launch):
// round_x != 0   the eager chain: quotient and floor live in the tensor's own element type, so both are rounded to it
//                (clamp(min=eps) on a bf16 tensor compares with eps rounded to bf16)
// round_x == 0   quotient and floor stay in fp32: what a code generator that fuses the chain leaves of it
//                (the reference's forward carries a torch.compile decorator, dax/quant/nn/dynamic/linear.py:143)
template <int XT>
__device__ __forceinline__ float scale_from_amax_bits_rt(uint32_t amax_bits, float qmax, float eps, int round_x) {
    float a = x_bits_to_f32<XT>(amax_bits);
    float s = a / qmax;
    if (round_x) {
        s = round_to_x<XT>(s);
        eps = round_to_x<XT>(eps);
    }
    return max_nan(s, eps);
}

// Wavefront-wide reductions with DPP (data-parallel primitives: the partner lane's value is an operand
// modifier of the VALU instruction, no trip through the LDS crossbar as with ds_bpermute): four steps
// give every lane the result of its row of 16 lanes, the four row results are then read as scalars.
#define DAXQ_DPP_QUAD_SWAP1 0xB1   /* quad_perm [1,0,3,2] */
#define DAXQ_DPP_QUAD_SWAP2 0x4E   /* quad_perm [2,3,0,1] */
#define DAXQ_DPP_HALF_MIRROR 0x141 /* lane i <-> 7 - i within 8 */
#define DAXQ_DPP_ROW_MIRROR 0x140  /* lane i <-> 15 - i within 16 */

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
}

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    uint32_t o;
    o = dpp_u32<DAXQ_DPP_QUAD_SWAP1>(v); v = v > o ? v : o;
    o = dpp_u32<DAXQ_DPP_QUAD_SWAP2>(v); v = v > o ? v : o;
    o = dpp_u32<DAXQ_DPP_HALF_MIRROR>(v); v = v > o ? v : o;
    o = dpp_u32<DAXQ_DPP_ROW_MIRROR>(v); v = v > o ? v : o;
    const uint32_t r0 = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), r1 = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
    const uint32_t r2 = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), r3 = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    const uint32_t a = r0 > r1 ? r0 : r1, b = r2 > r3 ? r2 : r3;
    return a > b ? a : b;
}

// fp32 sum over the wavefront, the same value in every lane (fixed order: deterministic)
__device__ __forceinline__ float wave_sum_f32(float x) {
    uint32_t v = __float_as_uint(x);
    v = __float_as_uint(__uint_as_float(v) + __uint_as_float(dpp_u32<DAXQ_DPP_QUAD_SWAP1>(v)));
    v = __float_as_uint(__uint_as_float(v) + __uint_as_float(dpp_u32<DAXQ_DPP_QUAD_SWAP2>(v)));
    v = __float_as_uint(__uint_as_float(v) + __uint_as_float(dpp_u32<DAXQ_DPP_HALF_MIRROR>(v)));
    v = __float_as_uint(__uint_as_float(v) + __uint_as_float(dpp_u32<DAXQ_DPP_ROW_MIRROR>(v)));
    const float r0 = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)v, 0));
    const float r1 = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)v, 16));
    const float r2 = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)v, 32));
    const float r3 = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)v, 48));
    return (r0 + r1) + (r2 + r3);
}

// clamp(rint(x * inv), -128, 127) as the low byte of a float: the product is clamped first (same result, the
// bounds are integers) and 1.5 * 2^23 is added, which rounds it to an integer, half to even, in the low mantissa
// bits; those bits are the two's-complement value.  Two operations fewer than round + convert.
// CLAMP = false: a row quantised with its own bf16-rounded (or fp32) scale of abs-max / 127 never leaves [-127.4, 127.4]
// (the rounding of the scale moves x * inv at the row maximum by at most 2^-8 of it: checked for every bf16 abs-max), so
// the clamp is dead code there and is left out.  (A NaN product -- an infinite element of a row whose scale is infinite
// -- then gives the byte 0 instead of -128; such a row's output is non-finite through its scale either way.)
template <bool CLAMP = true>
__device__ __forceinline__ uint32_t q_i8_bits(float x, float inv) {
    float r = x * inv;
    if constexpr (CLAMP) r = fminf(fmaxf(r, -128.0f), 127.0f);
    else asm("" : "+v"(r));  // the product is rounded before the addition, as in the reference: no contraction into one fma
    return __float_as_uint(r + 12582912.0f);
}

// FMT: 0 = int8, 1 = OCP e4m3fn (max 448), 2 = OCP e5m2 (max 57344)
// x / s, correctly rounded, from the correctly rounded reciprocal inv = RN(1 / s) of the row: one multiply,
// the exact residual by fma, one correction (Markstein's sequence; it yields RN(x / s) unless the
// significand of s is all ones, which a scale whose low 16 bits are zero never has).  The reference's
// true division costs about ten instructions per element when spelled x / s.
// TRUE_DIV: spell the division out (leaf quantiser with an arbitrary fp32 scale, used once per weight).
// CLAMP = false: with the row's own scale of abs-max / qmax the quotient at the row maximum stays below qmax * (1 + 2^-8)
// (449.5 for e4m3fn, 57530 for e5m2: checked for every bf16 abs-max), which the cast's round-to-nearest-even takes to
// the format's largest finite value by itself (the next step up lies beyond 464 / 61440), so the clamp is left out.
template <int FMT, bool TRUE_DIV, bool CLAMP = true>
__device__ __forceinline__ float q_f8_pre(float x, float s, float inv) {
    constexpr float kMax = FMT == 2 ? 57344.0f : 448.0f;
    float v;
    if constexpr (TRUE_DIV) {
        v = x / s;  // IEEE division
    } else {
        const float q0 = x * inv;
        const float e = __builtin_fmaf(-q0, s, x);
        v = __builtin_copysignf(__builtin_fmaf(e, inv, q0), x);  // s > 0; keeps -0 for x = -0 (0 + -0 is +0 in the fma)
    }
    // With a scale from the caller a NaN element must stay NaN through the clamp, as in the reference, and become
    // the format's NaN byte; with the row's own scale a NaN element has already made that scale NaN.
    if constexpr (!CLAMP) return v;
    if constexpr (TRUE_DIV) return min_nan(max_nan(v, -kMax), kMax);
    return fminf(fmaxf(v, -kMax), kMax);
}

template <int FMT>
__device__ __forceinline__ int cvt_pk_f8(float a, float b, int old, bool hi) {
    if constexpr (FMT == 2)
        return hi ? __builtin_amdgcn_cvt_pk_bf8_f32(a, b, old, true) : __builtin_amdgcn_cvt_pk_bf8_f32(a, b, old, false);
    else
        return hi ? __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, true) : __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, false);
}

// 8 bf16 / fp16 values (one 16-byte chunk) -> 8 quantised bytes
template <int FMT, bool TRUE_DIV = false, int XT = DAXQ_BF16, bool CLAMP = true>
__device__ __forceinline__ uint2 quant_chunk(const uint4& v, float s, float inv) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint32_t o[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        float f0, f1, f2, f3;
        if constexpr (XT == DAXQ_BF16) {
            f0 = __uint_as_float(w[2 * h] << 16);
            f1 = __uint_as_float(w[2 * h] & 0xffff0000u);
            f2 = __uint_as_float(w[2 * h + 1] << 16);
            f3 = __uint_as_float(w[2 * h + 1] & 0xffff0000u);
        } else {
            f0 = x_bits_to_f32<XT>(w[2 * h] & 0xffffu);
            f1 = x_bits_to_f32<XT>(w[2 * h] >> 16);
            f2 = x_bits_to_f32<XT>(w[2 * h + 1] & 0xffffu);
            f3 = x_bits_to_f32<XT>(w[2 * h + 1] >> 16);
        }
        if (FMT != 0) {
            int p = cvt_pk_f8<FMT>(q_f8_pre<FMT, TRUE_DIV, CLAMP>(f0, s, inv), q_f8_pre<FMT, TRUE_DIV, CLAMP>(f1, s, inv), 0, false);
            p = cvt_pk_f8<FMT>(q_f8_pre<FMT, TRUE_DIV, CLAMP>(f2, s, inv), q_f8_pre<FMT, TRUE_DIV, CLAMP>(f3, s, inv), p, true);
            o[h] = (uint32_t)p;
        } else {
            // byte 0 of each of the four words: three v_perm_b32
            const uint32_t p01 = __builtin_amdgcn_perm(q_i8_bits<CLAMP>(f1, inv), q_i8_bits<CLAMP>(f0, inv), 0x0c0c0400u);
            const uint32_t p23 = __builtin_amdgcn_perm(q_i8_bits<CLAMP>(f3, inv), q_i8_bits<CLAMP>(f2, inv), 0x0c0c0400u);
            o[h] = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
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

// Streaming accesses of the row kernels: the bf16 row is read once and the quantised row is written once, so both
// go past the caches with the non-temporal hint (measured: the per-token quantiser runs 6 - 11 % faster, the GEMM
// that reads the result afterwards is unchanged).
typedef unsigned daxq_v4u __attribute__((ext_vector_type(4)));
typedef unsigned daxq_v2u __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 load_stream_16(const uint4* p) {
    const daxq_v4u t = __builtin_nontemporal_load(reinterpret_cast<const daxq_v4u*>(p));
    return make_uint4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ void store_stream_8(uint2* p, uint2 v) {
    const daxq_v2u t = {v.x, v.y};
    __builtin_nontemporal_store(t, reinterpret_cast<daxq_v2u*>(p));
}

}  // namespace daxq
