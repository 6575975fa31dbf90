// Issue rate of the GEMM epilogue's VALU instructions when a SIMD holds ONE wavefront, which is how the 256x256 GEMM
// kernels run (512 registers per lane).  Every wavefront loops over independent register-only instructions; the
// program prints the time per instruction and wavefront.  On an MI355X a lone wavefront issues one VALU instruction
// about every 8 cycles (3.2 ns at 2.4 GHz), dependent or not, and v_permlane16_swap every 12: the epilogue's ~1900
// (INT8) / ~1200 (FP8) instructions per wavefront therefore take about 6 / 4 us per tile.
//
//   valu_rate            prints one line per instruction
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define CHECK(x)                                                   \
    do {                                                           \
        hipError_t e = (x);                                        \
        if (e != hipSuccess) {                                     \
            fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e)); \
            return 1;                                              \
        }                                                          \
    } while (0)

enum { MUL, ADD, CVT_I32, CVT_PK_BF16, PERMLANE16_SWAP, SHIFT_AND, ACC_READ, MUL_DEPENDENT };

template <int OP>
__global__ __launch_bounds__(256) void spin(int* out, int iters, float seed) {
    float a0 = seed, a1 = seed + 1, a2 = seed + 2, a3 = seed + 3, a4 = seed + 4, a5 = seed + 5, a6 = seed + 6, a7 = seed + 7;
    unsigned u0 = (unsigned)seed, u1 = u0 + 1, u2 = u0 + 2, u3 = u0 + 3;
    for (int it = 0; it < iters; ++it) {
        if constexpr (OP == MUL)
            asm volatile("v_mul_f32 %0, %0, %0\n v_mul_f32 %1, %1, %1\n v_mul_f32 %2, %2, %2\n v_mul_f32 %3, %3, %3\n"
                         "v_mul_f32 %4, %4, %4\n v_mul_f32 %5, %5, %5\n v_mul_f32 %6, %6, %6\n v_mul_f32 %7, %7, %7"
                         : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7));
        else if constexpr (OP == ADD)
            asm volatile("v_add_f32 %0, %0, %1\n v_add_f32 %1, %1, %2\n v_add_f32 %2, %2, %3\n v_add_f32 %3, %3, %4\n"
                         "v_add_f32 %4, %4, %5\n v_add_f32 %5, %5, %6\n v_add_f32 %6, %6, %7\n v_add_f32 %7, %7, %0"
                         : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7));
        else if constexpr (OP == CVT_I32)
            asm volatile("v_cvt_f32_i32 %0, %0\n v_cvt_f32_i32 %1, %1\n v_cvt_f32_i32 %2, %2\n v_cvt_f32_i32 %3, %3\n"
                         "v_cvt_f32_i32 %4, %4\n v_cvt_f32_i32 %5, %5\n v_cvt_f32_i32 %6, %6\n v_cvt_f32_i32 %7, %7"
                         : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7));
        else if constexpr (OP == CVT_PK_BF16)
            asm volatile("v_cvt_pk_bf16_f32 %0, %0, %1\n v_cvt_pk_bf16_f32 %1, %1, %2\n v_cvt_pk_bf16_f32 %2, %2, %3\n"
                         "v_cvt_pk_bf16_f32 %3, %3, %4\n v_cvt_pk_bf16_f32 %4, %4, %5\n v_cvt_pk_bf16_f32 %5, %5, %6\n"
                         "v_cvt_pk_bf16_f32 %6, %6, %7\n v_cvt_pk_bf16_f32 %7, %7, %0"
                         : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7));
        else if constexpr (OP == PERMLANE16_SWAP)
            asm volatile("v_permlane16_swap_b32 %0, %1\n v_permlane16_swap_b32 %2, %3\n v_permlane16_swap_b32 %0, %1\n"
                         "v_permlane16_swap_b32 %2, %3\n v_permlane16_swap_b32 %0, %1\n v_permlane16_swap_b32 %2, %3\n"
                         "v_permlane16_swap_b32 %0, %1\n v_permlane16_swap_b32 %2, %3"
                         : "+v"(u0), "+v"(u1), "+v"(u2), "+v"(u3));
        else if constexpr (OP == SHIFT_AND)
            asm volatile("v_lshlrev_b32 %0, 16, %0\n v_and_b32 %1, 0xffff0000, %1\n v_lshlrev_b32 %2, 16, %2\n"
                         "v_and_b32 %3, 0xffff0000, %3\n v_lshlrev_b32 %0, 16, %0\n v_and_b32 %1, 0xffff0000, %1\n"
                         "v_lshlrev_b32 %2, 16, %2\n v_and_b32 %3, 0xffff0000, %3"
                         : "+v"(u0), "+v"(u1), "+v"(u2), "+v"(u3));
        else if constexpr (OP == ACC_READ)
            asm volatile("v_accvgpr_read_b32 %0, a0\n v_accvgpr_read_b32 %1, a0\n v_accvgpr_read_b32 %2, a0\n"
                         "v_accvgpr_read_b32 %3, a0\n v_accvgpr_read_b32 %4, a0\n v_accvgpr_read_b32 %5, a0\n"
                         "v_accvgpr_read_b32 %6, a0\n v_accvgpr_read_b32 %7, a0"
                         : "+v"(a0), "+v"(a1), "+v"(a2), "+v"(a3), "+v"(a4), "+v"(a5), "+v"(a6), "+v"(a7)
                         :
                         : "a0");
        else
            asm volatile("v_mul_f32 %0, %0, %0\n v_mul_f32 %0, %0, %0\n v_mul_f32 %0, %0, %0\n v_mul_f32 %0, %0, %0\n"
                         "v_mul_f32 %0, %0, %0\n v_mul_f32 %0, %0, %0\n v_mul_f32 %0, %0, %0\n v_mul_f32 %0, %0, %0"
                         : "+v"(a0));
    }
    const float s = a0 + a1 + a2 + a3 + a4 + a5 + a6 + a7 + (float)(u0 + u1 + u2 + u3);
    if (s == 12345.678f) out[0] = 1;  // keeps the loop alive; never true in practice
}

template <int OP>
static int run(const char* name, int* dev) {
    const int iters = 20000, per_iter = 8;
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    hipLaunchKernelGGL(spin<OP>, dim3(256), dim3(256), 0, 0, dev, 100, 1.0f);  // one wavefront per SIMD
    CHECK(hipEventRecord(e0));
    hipLaunchKernelGGL(spin<OP>, dim3(256), dim3(256), 0, 0, dev, iters, 1.0f);
    CHECK(hipEventRecord(e1));
    CHECK(hipDeviceSynchronize());
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    printf("%-24s %.2f ns per instruction and wavefront\n", name, ms * 1e6 / iters / per_iter);
    return 0;
}

int main() {
    int* dev = nullptr;
    CHECK(hipMalloc(&dev, 16));
    CHECK(hipMemset(dev, 0, 16));
    int rc = run<MUL>("v_mul_f32", dev) | run<ADD>("v_add_f32", dev) | run<CVT_I32>("v_cvt_f32_i32", dev) |
             run<CVT_PK_BF16>("v_cvt_pk_bf16_f32", dev) | run<PERMLANE16_SWAP>("v_permlane16_swap_b32", dev) |
             run<SHIFT_AND>("v_lshlrev_b32 / v_and_b32", dev) | run<ACC_READ>("v_accvgpr_read_b32", dev) |
             run<MUL_DEPENDENT>("v_mul_f32, dependent", dev);
    CHECK(hipFree(dev));
    return rc;
}
