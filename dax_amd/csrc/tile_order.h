// Banded tile order of the 256x256 GEMM kernels (gfx950: 8 XCDs of 32 CUs, workgroup ids dealt round-robin over the
// XCDs).  Plain C++ on purpose: the host-side check in tests/host compiles this file without the HIP headers.
#pragma once

#include <stdint.h>

#ifdef __HIPCC__
#define DAXQ_HOST_DEVICE __host__ __device__ __forceinline__
#else
#define DAXQ_HOST_DEVICE inline
#endif

namespace daxq {

// Banded order.  With workgroup ids dealt round-robin over 8 XCDs, the 32 consecutive local ids (pid / 8) of an XCD are
// what its 32 CUs run side by side; they form one patch of 32 / w tile rows x w tile columns, so the CUs that share an
// L2 share 32 / w activation panels and w weight panels whatever the tile counts are.  The tile grid is cut into column
// bands: main bands of width W (8 or 4; the kernels use 4: patches of 8 x 4), and for the columns left over one band per
// set bit of tiles_n % W (widths 4, 2, 1: patches of 8 x 4, 16 x 2, 32 x 1), so no slot is padding in the width.  The
// tile rows are cut into super-rows of 32, a super-row into steps of one main-patch height, and a step emits one patch of
// every main band followed by the patch of each narrow band that starts at that row.  Patch 8 * round + xcd goes to XCD
// xcd, so the eight XCDs of a round sit in eight consecutive entries: on the same activation rows and on different weight
// bands when there are at least eight.  Slots beyond a patch's tiles (below the last tile row) are padding: their
// workgroups exit at once.  A full super-row emits tiles_n patches.
DAXQ_HOST_DEVICE int banded_before(int s, int hmain, int nb_main, int rem) {  // patches of a super-row before step s
    int c = s * nb_main;
    for (int wj = 4; wj >= 1; wj >>= 1)
        if (rem & wj) c += (s * hmain * wj + 31) >> 5;  // ceil(s * hmain / (32 / wj))
    return c;
}
DAXQ_HOST_DEVICE bool tile_of_block_banded(int pid, int tiles_m, int tiles_n, int W, int& tm, int& tn) {
    const int xcd = pid & 7, local = pid >> 3, slot = local & 31;
    const int patch = (local >> 5) * 8 + xcd;
    const int hmain = 32 / W, nb_main = tiles_n / W, rem = tiles_n - nb_main * W;
    const int sr = patch / tiles_n, u = patch - sr * tiles_n;
    int s = W - 1;  // steps of a super-row: 32 / hmain = W
    while (s > 0 && banded_before(s, hmain, nb_main, rem) > u) --s;
    int v = u - banded_before(s, hmain, nb_main, rem);
    const int row0 = sr * 32 + s * hmain;
    int h = hmain, col0 = v * W;
    if (v >= nb_main) {
        v -= nb_main;
        col0 = nb_main * W;
        h = 0;
        for (int wj = 4; wj >= 1; wj >>= 1) {
            if (!(rem & wj)) continue;
            const int hj = 32 / wj;
            if ((s * hmain) % hj == 0) {
                if (v == 0) {
                    h = hj;
                    break;
                }
                --v;
            }
            col0 += wj;
        }
        if (h == 0) return false;  // beyond the step's patches (cannot happen for u < patches of the super-row)
    }
    tm = row0 + slot % h;
    tn = col0 + slot / h;
    return tm < tiles_m;
}
// Tile times the slowest XCD needs in the banded order: ceil(its tiles / 32 CUs).  Patches of the full super-rows hold
// 32 tiles each; only those of the last, partial super-row are counted one by one.
inline int64_t banded_xcd_rounds(int tiles_m, int tiles_n, int W) {
    const int hmain = 32 / W, nb_main = tiles_n / W, rem = tiles_n - nb_main * W;
    const int64_t full = (int64_t)(tiles_m >> 5) * tiles_n;
    int64_t load[8];
    for (int x = 0; x < 8; ++x) load[x] = (full / 8 + (x < full % 8 ? 1 : 0)) * 32;
    const int left = tiles_m & 31;
    int next = (int)(full % 8);
    for (int s = 0; s * hmain < left; ++s) {
        const int row = s * hmain, rows_main = left - row < hmain ? left - row : hmain;
        for (int b = 0; b < nb_main; ++b, next = (next + 1) & 7) load[next] += rows_main * W;
        for (int wj = 4; wj >= 1; wj >>= 1) {
            if (!(rem & wj) || row % (32 / wj)) continue;
            const int hj = 32 / wj;
            load[next] += (left - row < hj ? left - row : hj) * wj;
            next = (next + 1) & 7;
        }
    }
    int64_t most = 0;
    for (int x = 0; x < 8; ++x) most = load[x] > most ? load[x] : most;
    return (most + 31) / 32;
}
inline int64_t banded_grid(int tiles_m, int tiles_n, int W) {
    const int hmain = 32 / W, nb_main = tiles_n / W, rem = tiles_n - nb_main * W;
    const int left = tiles_m & 31;
    const int64_t patches = (int64_t)(tiles_m >> 5) * tiles_n + banded_before((left + hmain - 1) / hmain, hmain, nb_main, rem);
    return (patches + 7) / 8 * 256;
}

}  // namespace daxq
