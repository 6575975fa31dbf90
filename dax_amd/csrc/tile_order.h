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
// bands when there are at least eight.  A full super-row emits tiles_n patches.
// The last, partial super-row (tiles_m % 32 rows): whole steps of hmain rows as above; the r < hmain rows left under them
// form dense patches of r rows x (32 / r) columns over the main bands and over every narrow band that would start a
// patch at that row (the bands further right are still inside a patch that started higher up).  Slots beyond a patch's
// tiles are padding: their workgroups exit at once.
// (Cutting the patches of the last round further so that every XCD works in the launch's last tile time was measured
// in two forms, tile by tile and in pieces of consecutive rows: both slower than whole patches.)
struct BandedGrid {
    int tiles_m, tiles_n, W, hmain, nb_main, rem;
    int full_sr;               // whole super-rows
    int full_steps, r, wr;     // partial super-row: whole steps, rows left under them, width of their dense patches
    int dense_cols, dense_n;   // columns the dense patches cover, and their count
    int tail_before;           // patches of the partial super-row in front of the dense ones
    int patches;               // all patches of the grid (the launchers keep grids below 2^31 workgroups)
};
DAXQ_HOST_DEVICE int banded_before(int s, int hmain, int nb_main, int rem) {  // patches of a super-row before step s
    int c = s * nb_main;
    for (int wj = 4; wj >= 1; wj >>= 1)
        if (rem & wj) c += (s * hmain * wj + 31) >> 5;  // ceil(s * hmain / (32 / wj))
    return c;
}
DAXQ_HOST_DEVICE BandedGrid banded_make(int tiles_m, int tiles_n, int W) {
    BandedGrid g;
    g.tiles_m = tiles_m, g.tiles_n = tiles_n, g.W = W;
    g.hmain = 32 / W, g.nb_main = tiles_n / W, g.rem = tiles_n - g.nb_main * W;
    g.full_sr = tiles_m >> 5;
    const int left = tiles_m & 31;
    g.full_steps = left / g.hmain;
    g.r = left - g.full_steps * g.hmain;
    g.wr = g.r ? 32 / g.r : 0;
    g.dense_cols = g.nb_main * W;
    for (int wj = 4; wj >= 1; wj >>= 1)
        if ((g.rem & wj) && (g.full_steps * g.hmain) % (32 / wj) == 0) g.dense_cols += wj;
    g.dense_n = g.r ? (g.dense_cols + g.wr - 1) / g.wr : 0;
    g.tail_before = banded_before(g.full_steps, g.hmain, g.nb_main, g.rem);
    g.patches = g.full_sr * tiles_n + g.tail_before + g.dense_n;
    return g;
}
// Patch `patch` of the grid: slot s of it is tile (row0 + s % h, col0 + s / h) when s % h < rows and s / h < cols.
DAXQ_HOST_DEVICE bool banded_patch(const BandedGrid& g, int patch, int& row0, int& col0, int& h, int& rows, int& cols) {
    if (patch >= g.patches) return false;
    const int sr = patch / g.tiles_n, u = patch - sr * g.tiles_n;
    int s = g.W - 1;  // steps of a super-row: 32 / hmain = W
    if (sr == g.full_sr) {
        const int v = u - g.tail_before;
        if (v >= 0) {  // dense patches of the rows under the whole steps
            row0 = sr * 32 + g.full_steps * g.hmain;
            col0 = v * g.wr;
            h = rows = g.r;
            cols = g.dense_cols - col0 < g.wr ? g.dense_cols - col0 : g.wr;
            return true;
        }
        s = g.full_steps - 1;
    }
    while (s > 0 && banded_before(s, g.hmain, g.nb_main, g.rem) > u) --s;
    int v = u - banded_before(s, g.hmain, g.nb_main, g.rem);
    row0 = sr * 32 + s * g.hmain;
    h = g.hmain, col0 = v * g.W, cols = g.W;
    if (v >= g.nb_main) {
        v -= g.nb_main;
        col0 = g.nb_main * g.W;
        h = 0;
        for (int wj = 4; wj >= 1; wj >>= 1) {
            if (!(g.rem & wj)) continue;
            const int hj = 32 / wj;
            if ((s * g.hmain) % hj == 0) {
                if (v == 0) {
                    h = hj, cols = wj;
                    break;
                }
                --v;
            }
            col0 += wj;
        }
        if (h == 0) return false;  // beyond the step's patches (cannot happen for u < patches of the super-row)
    }
    rows = g.tiles_m - row0 < h ? g.tiles_m - row0 : h;
    return true;
}
DAXQ_HOST_DEVICE bool tile_of_block_banded(int pid, int tiles_m, int tiles_n, int W, int& tm, int& tn) {
    const BandedGrid g = banded_make(tiles_m, tiles_n, W);
    const int xcd = pid & 7, local = pid >> 3, slot = local & 31;
    int row0, col0, h, rows, cols;
    if (!banded_patch(g, (local >> 5) * 8 + xcd, row0, col0, h, rows, cols)) return false;
    const int r = slot % h, c = slot / h;
    tm = row0 + r;
    tn = col0 + c;
    return r < rows && c < cols;
}
inline int64_t banded_grid(int tiles_m, int tiles_n, int W) { return ((int64_t)banded_make(tiles_m, tiles_n, W).patches + 7) / 8 * 256; }
// Tile times the slowest XCD needs in the banded order: ceil(its tiles / 32 CUs).  Patches of the full super-rows hold
// 32 tiles each; those of the last, partial super-row are counted one by one.
inline int64_t banded_xcd_rounds(int tiles_m, int tiles_n, int W) {
    const BandedGrid g = banded_make(tiles_m, tiles_n, W);
    const int full = g.full_sr * tiles_n;  // patches of 32 tiles
    int64_t load[8];
    for (int x = 0; x < 8; ++x) load[x] = (int64_t)(full / 8 + (x < full % 8 ? 1 : 0)) * 32;
    for (int patch = full; patch < g.patches; ++patch) {
        int row0, col0, h, rows, cols;
        if (banded_patch(g, patch, row0, col0, h, rows, cols)) load[patch & 7] += rows * cols;
    }
    int64_t most = 0;
    for (int x = 0; x < 8; ++x) most = load[x] > most ? load[x] : most;
    return (most + 31) / 32;
}

}  // namespace daxq
