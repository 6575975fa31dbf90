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

// f32 -> bf16 bits, round to nearest even (finite inputs)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}

}  // namespace daxq
