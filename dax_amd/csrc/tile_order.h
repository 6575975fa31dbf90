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

// The same patches in an order that keeps an XCD on the same activation rows for as long as possible: the tile rows
// are cut into super-groups of lcm(4, 32 / w) rows (w = tiles_n % 8; 4 rows when w = 0), a super-group's patches
// follow one another (its 4-row groups across the 8-wide bands, then its remainder patches), and XCD x runs the
// x-th eighth of that sequence.  An activation panel is then fetched from HBM by one XCD and re-read only by that
// XCD, a few rounds later, as with the row-group order; the round-robin order above has two XCDs fetch it at the same
// time and comes back to it a whole band later.
struct PatchSeq {
    int sg_rows, per_sg, band_patches, n_sg, total;  // rows and patches of a super-group, its band patches, super-groups
};
DAXQ_HOST_DEVICE PatchSeq patch_sequence(int tiles_m, int tiles_n) {
    const int nb8 = tiles_n >> 3, rw = tiles_n & 7;
    PatchSeq q;
    int rp = 4;
    if (rw) rp = 32 / rw;
    // lcm(4, rp) for rp in {32, 16, 10, 8, 6, 5, 4}
    q.sg_rows = !rw ? 4 : (rp % 4 == 0 ? rp : (rp % 2 == 0 ? 2 * rp : 4 * rp));
    q.band_patches = nb8 * (q.sg_rows >> 2);
    q.per_sg = q.band_patches + (rw ? q.sg_rows / rp : 0);
    q.n_sg = (tiles_m + q.sg_rows - 1) / q.sg_rows;
    q.total = q.n_sg * q.per_sg;
    return q;
}
DAXQ_HOST_DEVICE bool tile_of_block_supergroups(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
    const PatchSeq q = patch_sequence(tiles_m, tiles_n);
    const int xcd = pid & 7, local = pid >> 3, round = local >> 5, slot = local & 31;
    const int first = (int)(((int64_t)xcd * q.total) >> 3), end = (int)(((int64_t)(xcd + 1) * q.total) >> 3);
    const int s = first + round;
    if (s >= end) return false;
    const int nb8 = tiles_n >> 3, rw = tiles_n & 7;
    const int sg = s / q.per_sg, w = s - sg * q.per_sg;
    if (w < q.band_patches) {
        const int gi = w / nb8, b = w - gi * nb8;
        tm = sg * q.sg_rows + gi * 4 + (slot & 3);
        tn = b * 8 + (slot >> 2);
        return tm < tiles_m;
    }
    const int rp = 32 / rw, qi = w - q.band_patches;
    const int r = slot / rw, c = slot - r * rw;
    tm = sg * q.sg_rows + qi * rp + r;
    tn = nb8 * 8 + c;
    return r < rp && tm < tiles_m;
}
inline int64_t supergroups_grid(int tiles_m, int tiles_n) {
    const PatchSeq q = patch_sequence(tiles_m, tiles_n);
    int most = 0;
    for (int x = 0; x < 8; ++x) {
        const int n = (int)((((int64_t)(x + 1) * q.total) >> 3) - (((int64_t)x * q.total) >> 3));
        most = n > most ? n : most;
    }
    return (int64_t)most * 256;
}

}  // namespace daxq
