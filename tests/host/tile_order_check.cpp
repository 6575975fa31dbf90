// Host-side check of the banded tile order (dax_amd/csrc/tile_order.h): for every tile grid up to 320 x 72, and for
// sampled grids far beyond (tile rows up to 40000, tile columns up to 4096: the range the library's choice by shape
// admits), the launch of banded_grid() workgroups computes every tile exactly once, padding slots map to no tile, and
// the 32 slots that one XCD runs side by side lie in one patch of at most 32 tiles, at most 8 columns wide (wider only
// in the dense patches of the last tile rows).  Built by
// __graft_entry__.build() with the host compiler; run by tests/test_abi_and_host.py.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../dax_amd/csrc/tile_order.h"

static long check_grid(int tiles_m, int tiles_n, int W) {
    long bad = 0;
    std::vector<unsigned char> seen((size_t)tiles_m * tiles_n, 0);
    const int64_t grid = daxq::banded_grid(tiles_m, tiles_n, W);
    if (grid % 256 != 0 || grid < (int64_t)tiles_m * tiles_n || grid > 0x7fffffff) return 1;
    for (int64_t base = 0; base < grid; base += 256)
        for (int xcd = 0; xcd < 8; ++xcd) {
            int lo_m = 1 << 30, hi_m = -1, lo_n = 1 << 30, hi_n = -1;
            for (int slot = 0; slot < 32; ++slot) {
                const int pid = (int)base + slot * 8 + xcd;  // the 32 consecutive local ids of this XCD
                int tm = -1, tn = -1;
                if (!daxq::tile_of_block_banded(pid, tiles_m, tiles_n, W, tm, tn)) continue;
                if (tm < 0 || tm >= tiles_m || tn < 0 || tn >= tiles_n) {
                    ++bad;
                    continue;
                }
                if (seen[(size_t)tm * tiles_n + tn]++) ++bad;  // computed twice
                lo_m = tm < lo_m ? tm : lo_m;
                hi_m = tm > hi_m ? tm : hi_m;
                lo_n = tn < lo_n ? tn : lo_n;
                hi_n = tn > hi_n ? tn : hi_n;
            }
            if (hi_m >= 0) {
                const int rows = hi_m - lo_m + 1, cols = hi_n - lo_n + 1;
                // panels shared inside an XCD: rows + cols of one patch; wider than 8 only in the rows under the last whole step
                if (rows * cols > 32 || (cols > 8 && tiles_m - lo_m >= 8)) ++bad;
            }
        }
    for (unsigned char v : seen) bad += v != 1;  // never computed
    return bad;
}

int main() {
    long grids = 0, bad = 0;
    for (int W : {8, 4})
        for (int tiles_m = 1; tiles_m <= 320; tiles_m += (tiles_m < 48 ? 1 : 17))
            for (int tiles_n = 1; tiles_n <= 72; ++tiles_n, ++grids) bad += check_grid(tiles_m, tiles_n, W);
    // far beyond the benchmark's grids: many tile rows (M in the millions), many tile columns (N up to a million)
    for (int tiles_m : {321, 1000, 4097, 40000})
        for (int tiles_n = 73; tiles_n <= 4096; tiles_n += 97, ++grids) {
            if ((int64_t)tiles_m * tiles_n > 60000000) continue;
            bad += check_grid(tiles_m, tiles_n, 4);
        }
    for (int tiles_n : {20, 54, 60, 255, 256, 257, 1023, 4095, 4096}) {
        bad += check_grid(100003, tiles_n > 512 ? 512 : tiles_n, 4);
        bad += check_grid(33, tiles_n, 4);
        grids += 2;
    }
    // banded_xcd_rounds against a count of the tiles that tile_of_block_banded gives every XCD
    for (int W : {8, 4})
        for (int tiles_m = 1; tiles_m <= 300; tiles_m += (tiles_m < 70 ? 1 : 23))
            for (int tiles_n = 1; tiles_n <= 72; ++tiles_n) {
                long load[8] = {0};
                const int64_t grid = daxq::banded_grid(tiles_m, tiles_n, W);
                for (int64_t pid = 0; pid < grid; ++pid) {
                    int tm, tn;
                    if (daxq::tile_of_block_banded((int)pid, tiles_m, tiles_n, W, tm, tn)) ++load[pid & 7];
                }
                long most = 0;
                for (long v : load) most = v > most ? v : most;
                ++grids;
                bad += daxq::banded_xcd_rounds(tiles_m, tiles_n, W) != (most + 31) / 32;
            }
    // 8 x 4 patches: no more rounds of tiles than the tile count itself needs on the benchmark launches
    const long want[3][2] = {{296, 20}, {296, 60}, {296, 54}};
    for (auto& w : want) bad += daxq::banded_grid((int)w[0], (int)w[1], 4) != (w[0] * w[1] + 255) / 256 * 256;
    std::printf("%ld tile grids checked, %ld errors\n", grids, bad);
    return bad ? 1 : 0;
}
