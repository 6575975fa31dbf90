// Host-side check of the patch tile orders (dax_amd/csrc/tile_order.h: patch-aligned, super-groups, banded, swept): for
// every tile grid up to 320 x 72 the launch of *_grid() workgroups computes every tile exactly once, padding slots map
// to no tile, and the 32 slots that one XCD runs side by side lie in one patch of at most 32 tiles, 8 columns wide.  Built by
// __graft_entry__.build() with the host compiler; run by tests/test_abi_and_host.py.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../dax_amd/csrc/tile_order.h"

template <class Map, class Grid>
static long check_order(Map map, Grid grid_of, long& grids) {
    long bad = 0;
    for (int tiles_m = 1; tiles_m <= 320; tiles_m += (tiles_m < 48 ? 1 : 17))
        for (int tiles_n = 1; tiles_n <= 72; ++tiles_n) {
            ++grids;
            std::vector<int> seen((size_t)tiles_m * tiles_n, 0);
            const int64_t grid = grid_of(tiles_m, tiles_n);
            if (grid % 256 != 0 || grid < (int64_t)tiles_m * tiles_n) ++bad;
            for (int64_t base = 0; base < grid; base += 256)
                for (int xcd = 0; xcd < 8; ++xcd) {
                    int lo_m = 1 << 30, hi_m = -1, lo_n = 1 << 30, hi_n = -1;
                    for (int slot = 0; slot < 32; ++slot) {
                        const int pid = (int)base + slot * 8 + xcd;  // the 32 consecutive local ids of this XCD
                        int tm = -1, tn = -1;
                        if (!map(pid, tiles_m, tiles_n, tm, tn)) continue;
                        if (tm < 0 || tm >= tiles_m || tn < 0 || tn >= tiles_n) {
                            ++bad;
                            continue;
                        }
                        ++seen[(size_t)tm * tiles_n + tn];
                        lo_m = tm < lo_m ? tm : lo_m;
                        hi_m = tm > hi_m ? tm : hi_m;
                        lo_n = tn < lo_n ? tn : lo_n;
                        hi_n = tn > hi_n ? tn : hi_n;
                    }
                    if (hi_m >= 0) {
                        const int rows = hi_m - lo_m + 1, cols = hi_n - lo_n + 1;
                        if (cols > 8 || rows * cols > 32) ++bad;  // panels shared inside an XCD: rows + cols of one patch
                    }
                }
            for (int v : seen) bad += v != 1;
        }
    return bad;
}

int main() {
    long grids = 0;
    long bad = check_order([](int pid, int a, int b, int& tm, int& tn) { return daxq::tile_of_block_patched(pid, a, b, tm, tn); },
                           [](int a, int b) { return daxq::patched_grid(a, b); }, grids);
    bad += check_order([](int pid, int a, int b, int& tm, int& tn) { return daxq::tile_of_block_supergroups(pid, a, b, tm, tn); },
                       [](int a, int b) { return daxq::supergroups_grid(a, b); }, grids);
    for (int W : {8, 4})
        bad += check_order([W](int pid, int a, int b, int& tm, int& tn) { return daxq::tile_of_block_banded(pid, a, b, W, tm, tn); },
                           [W](int a, int b) { return daxq::banded_grid(a, b, W); }, grids);
    for (int W : {8, 4})
        bad += check_order([W](int pid, int a, int b, int& tm, int& tn) { return daxq::tile_of_block_swept(pid, a, b, W, tm, tn); },
                           [W](int a, int b) { return daxq::swept_grid(a, b, W); }, grids);
    // the four benchmark launches: grid sizes and padding
    const long want[3][3] = {{296, 20, 6144}, {296, 60, 17920}, {296, 54, 16128}};
    for (auto& w : want) bad += daxq::patched_grid((int)w[0], (int)w[1]) != w[2];
    const long want_sg[3] = {6144, 17920, 16384};  // 296 x 54: super-groups of 20 rows, the last one holds 6 empty patches
    for (int i = 0; i < 3; ++i) bad += daxq::supergroups_grid((int)want[i][0], (int)want[i][1]) != want_sg[i];
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
    // banded order, 8 x 4 patches: no more rounds of tiles than the tile count itself needs on the four benchmark launches
    for (auto& w : want) bad += daxq::banded_grid((int)w[0], (int)w[1], 4) != (w[0] * w[1] + 255) / 256 * 256;
    std::printf("%ld tile grids checked, %ld errors\n", grids, bad);
    return bad ? 1 : 0;
}
