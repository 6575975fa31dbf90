// Patch-aligned tile order of the 256x256 GEMM kernels (gfx950: 8 XCDs of 32 CUs, workgroup ids dealt round-robin over
// the XCDs).  Plain C++ on purpose: the host-side check in tests/host compiles this file without the HIP headers.
#pragma once

#include <stdint.h>

#ifdef __HIPCC__
#define DAXQ_HOST_DEVICE __host__ __device__ __forceinline__
#else
#define DAXQ_HOST_DEVICE inline
#endif

namespace daxq {

// Patch-aligned order.  The tile grid is cut into column bands, 8 tile columns wide plus one
// band for the remaining tiles_n % 8 columns, and each band into patches of 32 slots: 4 rows x 8 columns, or
// (32 / w) rows x w columns in the remainder band.  A patch is what the 32 CUs of one XCD run side by side: with
// workgroup ids dealt round-robin over 8 XCDs, the 32 consecutive local ids (pid / 8) of an XCD form one patch, so
// the CUs that share an L2 always share 4 activation panels and 8 weight panels (or 32 / w and w), whatever the tile
// counts are.  Slots beyond a patch's tiles are padding: their workgroups exit at once.
// Returns false for a padding slot.
DAXQ_HOST_DEVICE bool tile_of_block_patched(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int xcd = pid & 7, local = pid >> 3;
    const int patch = (local >> 5) * 8 + xcd, slot = local & 31;
    const int nb8 = tiles_n >> 3, rw = tiles_n & 7;
    const int p8 = nb8 * ((tiles_m + 3) >> 2);
    if (patch < p8) {
        const int g = patch / nb8, b = patch - g * nb8;
        tm = g * 4 + (slot & 3);
        tn = b * 8 + (slot >> 2);
        return tm < tiles_m;
    }
    if (rw == 0) return false;
    const int rp = 32 / rw, q = patch - p8;
    const int r = slot / rw, c = slot - r * rw;
    tm = q * rp + r;
    tn = nb8 * 8 + c;
    return r < rp && tm < tiles_m;
}

// workgroups of a launch in that order: 256 per round of patches (32 slots x 8 XCDs)
inline int64_t patched_grid(int tiles_m, int tiles_n) {
    const int nb8 = tiles_n >> 3, rw = tiles_n & 7;
    int64_t patches = (int64_t)nb8 * ((tiles_m + 3) >> 2);
    if (rw) {
        const int rp = 32 / rw;
        patches += (tiles_m + rp - 1) / rp;
    }
    return (patches + 7) / 8 * 256;
}

}  // namespace daxq
