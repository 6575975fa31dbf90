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

// Banded order.  Same idea as the patch-aligned order (32 slots of an XCD = one patch of 32 / w rows x w columns), with
// two changes that keep the XCDs on DIFFERENT weight panels at any one time:
//   * the columns left over by the main bands (width W = 8 or 4) form one band per set bit of tiles_n % W (widths 4, 2,
//     1: patches of 8 x 4, 16 x 2, 32 x 1), so no slot is padding in the width;
//   * those narrow bands are woven into the sequence instead of being appended to it: the tile rows are cut into
//     super-rows of 32, a super-row into steps of one main-patch height, and a step emits one patch of every main band
//     followed by the patch of each narrow band that starts at that row.  Patch 8 * round + xcd goes to XCD xcd, so
//     the eight XCDs of a round sit in eight consecutive entries: different bands when there are at least eight.
// A full super-row emits tiles_n patches.
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

// Swept order.  Patches of 32 / W rows x W columns again, but every XCD keeps to itself: the patches are listed row
// block by row block (a row block = one patch height of tile rows, nb = ceil(tiles_n / W) patches), XCD x owns the
// x-th eighth of that list and walks through it, so that consecutive patches of an XCD share their activation panels
// and no activation panel is ever wanted by two XCDs at the same time.  Inside a row block the bands are visited in
// an order rotated per XCD, such that at any one time XCD x is about x * nb / 8 bands ahead of XCD 0: the eight
// XCDs read different weight panels.  The last band may be narrower than W and the last row block shorter than a
// patch: those slots are padding.
DAXQ_HOST_DEVICE int swept_cut(int x, int total) { return (int)(((int64_t)x * total) >> 3); }
DAXQ_HOST_DEVICE bool tile_of_block_swept(int pid, int tiles_m, int tiles_n, int W, int& tm, int& tn) {
    const int xcd = pid & 7, local = pid >> 3, round = local >> 5, slot = local & 31;
    const int H = 32 / W, nb = (tiles_n + W - 1) / W, rbs = (tiles_m + H - 1) / H, total = nb * rbs;
    const int i = swept_cut(xcd, total) + round;
    if (i >= swept_cut(xcd + 1, total)) return false;
    const int rb = i / nb, j = i - rb * nb;
    int owner = xcd;  // the XCD that owns the first patch of this row block decides the rotation
    while (owner > 0 && swept_cut(owner, total) > rb * nb) --owner;
    int rot = (owner * nb) / 8 - swept_cut(owner, total) % nb;
    rot = rot < 0 ? rot + nb : rot;
    int band = j + rot;
    band = band >= nb ? band - nb : band;
    tm = rb * H + slot % H;
    tn = band * W + slot / H;
    return tm < tiles_m && tn < tiles_n;
}
inline int64_t swept_grid(int tiles_m, int tiles_n, int W) {
    const int H = 32 / W, nb = (tiles_n + W - 1) / W, rbs = (tiles_m + H - 1) / H, total = nb * rbs;
    int most = 0;
    for (int x = 0; x < 8; ++x) {
        const int n = swept_cut(x + 1, total) - swept_cut(x, total);
        most = n > most ? n : most;
    }
    return (int64_t)most * 256;
}

}  // namespace daxq
