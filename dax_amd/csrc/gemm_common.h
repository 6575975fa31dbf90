// Types and helpers shared by the W8A8 GEMM kernels (gfx950).
#pragma once

#include <atomic>

#include "daxq_common.h"
#include "tile_order.h"

namespace daxq {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));

#define DAXQ_LDS __attribute__((address_space(3)))
#define DAXQ_GLOBAL __attribute__((address_space(1)))

template <bool FP8>
struct AccT {
    typedef v16i type;
};
template <>
struct AccT<true> {
    typedef v16f type;
};

struct GemmArgs {
    const uint8_t* a;  // xq [m, k]
    const uint8_t* b;  // wq [n, k]
    const float* sx;   // [m]
    const float* sw;   // [n]
    const uint16_t* bias;  // bf16 [n] or null
    uint16_t* out;     // bf16 [m, n]
    void* acc;         // int32 / fp32 [m, n] dump or null
    int64_t lda, ldb, ldo, ldacc;
    int m, n, k;
    int tiles_m, tiles_n;
    int gm;  // depth (in tile rows) of the groups the tile order walks through
    // tile order of the 256x256 kernels: 0 = groups of gm tile rows, 1 = banded patches of 8 x 4 tiles (tile_order.h)
    int order;
    int out_kind;  // element type of out and bias: DAXQ_BF16 / DAXQ_F16 / DAXQ_F32
    // split-K launches only: K is cut into `splits` equal ranges, one workgroup each; partial accumulators go to
    // `partials` ([tile][split][64 KiB]) and the workgroup that arrives last at `counters[tile]` adds them up
    int splits;
    int32_t* counters;
    void* partials;
    // A launch of 256x256 tiles with few rounds of workgroups leaves most CUs idle during its last, partial round.
    // Such a launch runs the tiles of that round in smaller pieces with a CU each: with `grid` > 0 only the first
    // `grid` workgroups of the launch compute whole tiles of the row-group order (the whole rounds), and the
    // workgroups behind them compute the 128x128 quadrants (four workgroups per tile) or the 256x128 halves (two) of
    // the tiles from id quad_base - 1 on (tiles_m / tiles_n count 256x256 tiles).  0 = off.
    int grid, quad_base;
};

// FP8 operand formats of a launch as one template parameter: bit 0 = activations are e5m2, bit 1 = weights are e5m2
// (the format selects of the f8f6f4 MFMA are instruction immediates)
constexpr int kF8XE5 = 1, kF8WE5 = 2;

// Raises a kernel's dynamic LDS limit once per device.  `done` is the caller's per-kernel bit mask of the devices
// already set up (a race between two threads sets the same attribute twice).
inline int ensure_dynamic_lds(const void* kern, int bytes, std::atomic<uint64_t>& done) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return fail(DAXQ_ERR_LAUNCH, "hipGetDevice failed");
    const uint64_t bit = dev < 64 ? (uint64_t)1 << dev : 0;
    if (done.load(std::memory_order_acquire) & bit) return DAXQ_OK;
    hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return fail(DAXQ_ERR_LAUNCH, "hipFuncSetAttribute(%d bytes LDS): %s", bytes, hipGetErrorString(e));
    done.fetch_or(bit, std::memory_order_release);
    return DAXQ_OK;
}

// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding: vmcnt in bits 3:0 and 15:14,
// expcnt 6:4 and lgkmcnt 11:8 left at their maxima)
constexpr int vmcnt_imm(int n) { return (n & 15) | ((n >> 4) << 14) | 0x0070 | 0x0f00; }

// and-mask that turns an s_waitcnt immediate into one that also waits for lgkmcnt == 0
constexpr int lgkmcnt0_mask() { return ~0x0f00; }
// ... for lgkmcnt <= n (n < 16)
constexpr int lgkmcnt_mask(int n) { return ~0x0f00 | (n << 8); }

__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// Maps the flat workgroup id to an output tile.  Hardware deals consecutive ids round-robin
// over the 8 XCDs; give each XCD one contiguous range of the tile sequence, and order the
// sequence in groups of GM tile rows so a range covers a near-square patch.
__device__ __forceinline__ void tile_of_block(int GM, int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int nt = tiles_m * tiles_n;
    const int xcd = pid & 7, q = nt >> 3, r = nt & 7;
    const int id = xcd * q + (xcd < r ? xcd : r) + (pid >> 3);
    const int per_group = GM * tiles_n;
    const int g = id / per_group;
    const int first = g * GM;
    const int gsz = (tiles_m - first) < GM ? (tiles_m - first) : GM;
    const int in_g = id - g * per_group;
    tm = first + in_g % gsz;
    tn = in_g / gsz;
}

}  // namespace daxq
