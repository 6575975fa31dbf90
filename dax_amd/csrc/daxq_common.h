// Shared host/device helpers for the daxq kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/daxq.h"

namespace daxq {

// thread-local error text behind daxq_last_error()
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);

// checks a launch and converts a HIP error into DAXQ_ERR_LAUNCH
int check_launch(const char* what);

constexpr float kEps = 1.1920928955078125e-07f;  // 2^-23 = torch.finfo(float32).eps

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }
__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
// two floats rounded to fp16 (nearest even; overflow gives infinity, as a cast does), lo in the low half
__device__ __forceinline__ uint32_t pack_f16_rne(float lo, float hi) {
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)lo) | ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)hi) << 16);
}

// max / min that give NaN when either operand is NaN, like torch.max / torch.min / torch.clamp on tensors
// (fmaxf and fminf drop a NaN operand, which would turn a poisoned row into finite garbage)
__device__ __forceinline__ float max_nan(float a, float b) { return (a != a || a > b) ? a : b; }
__device__ __forceinline__ float min_nan(float a, float b) { return (a != a || a < b) ? a : b; }

// f32 -> bf16 bits, round to nearest even (finite inputs)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}

// two f32 -> two bf16 in one word (lo = first), round to nearest even: v_cvt_pk_bf16_f32
typedef __bf16 daxq_bf16x2 __attribute__((ext_vector_type(2)));
typedef float daxq_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16_rne(float lo, float hi) {
    daxq_f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, daxq_bf16x2));
}

}  // namespace daxq
