// Host-side check of the bf6 GEMM's tile order (dsaquant_amd/csrc/vdmq_bf6_tilemap.h): for every grid of output tiles
// in a range, both main super-tile shapes, edges regrouped or not, and the three ways the super-tile sequence is dealt to the XCDs, each tile is
// taken exactly once, by a place inside the grid, and the closed-form tile counts agree with the enumeration.  Super-tiles
// of 32 places (the 256 x 256 tiles' kernels) on the full range; of 1 ... 64 places (what the launcher picks for the
// few 128 x 128 tiles of a small problem) on a smaller one.
// Prints "ok <cases>" or the first disagreement; built and run by tests/test_host.py.
#include <cstdio>
#include <vector>

#include "vdmq_bf6_tilemap.h"

using namespace vdmq;

static int check(int tiles_m, int tiles_n, int gn_log2, int mode, bool regroup, int per_log2 = 5) {
    const int per = 1 << per_log2;
    Bf6TileMap tm;
    bf6_tilemap_shape(tm, tiles_m, tiles_n, per_log2, gn_log2, regroup);
    tm.contig = 0;
    int rounds = (tm.total_super + kBf6Xcds - 1) / kBf6Xcds;
    if (mode != 0) rounds = bf6_tilemap_runs(tm, mode == 1);
    if (tm.total_super != tm.n_main + tm.n_edge_n + tm.n_edge_m) return 1;
    if (bf6_tilemap_tiles_before(tm, 0) != 0 || bf6_tilemap_tiles_before(tm, tm.total_super) != int64_t(tiles_m) * tiles_n) return 2;
    if (mode != 0) {
        if (tm.start[0] != 0 || tm.start[kBf6Xcds] != tm.total_super) return 3;
        for (int x = 0; x < kBf6Xcds; ++x)
            if (tm.start[x] > tm.start[x + 1] || tm.start[x + 1] - tm.start[x] > rounds) return 4;
    }
    std::vector<int> seen(size_t(tiles_m) * tiles_n, 0), super_seen(tm.total_super, 0);
    for (int xcd = 0; xcd < kBf6Xcds; ++xcd)
        for (int seq = 0; seq <= rounds; ++seq) {
            const int st = bf6_tilemap_super(tm, xcd, seq);
            if (st < 0) continue;
            if (seq == rounds || st >= tm.total_super) return 5; /* the launch has `rounds` rounds */
            ++super_seen[st];
            int here = 0;
            for (int place = 0; place < per; ++place) {
                int m = -7, n = -7;
                if (!bf6_tilemap_locate(tm, st, place, m, n)) continue;
                if (m < 0 || m >= tiles_m || n < 0 || n >= tiles_n) return 6;
                ++seen[size_t(m) * tiles_n + n];
                ++here;
            }
            if (here == 0) return 7; /* no super-tile is empty */
            if (bf6_tilemap_tiles_before(tm, st + 1) - bf6_tilemap_tiles_before(tm, st) != here) return 8;
        }
    for (int v : seen)
        if (v != 1) return 9;
    for (int v : super_seen)
        if (v != 1) return 10;
    if (mode == 2 && rounds != (tm.total_super + kBf6Xcds - 1) / kBf6Xcds) return 11;
    return 0;
}

int main() {
    long cases = 0;
    const int big[][2] = {{296, 60}, {296, 54}, {296, 20}, {107, 56}, {107, 36}, {107, 12}, {128, 35}, {128, 18}, {128, 6}, {2, 40}, {1000, 3}, {3, 1000}, {4096, 1}, {1, 4096}};
    for (int variant = 0; variant < 4; ++variant)
        for (int mode = 0; mode < 3; ++mode) {
            const int gn_log2 = 1 + variant % 2;
            const bool regroup = variant >= 2;
            for (int m = 1; m <= 72; ++m)
                for (int n = 1; n <= 72; ++n, ++cases)
                    if (int e = check(m, n, gn_log2, mode, regroup)) return std::printf("tiles %d x %d, columns per group %d, regrouped %d, mode %d: check %d failed\n", m, n, 1 << gn_log2, regroup, mode, e), 1;
            for (auto &b : big) {
                ++cases;
                if (int e = check(b[0], b[1], gn_log2, mode, regroup)) return std::printf("tiles %d x %d, columns per group %d, regrouped %d, mode %d: check %d failed\n", b[0], b[1], 1 << gn_log2, regroup, mode, e), 1;
            }
        }
    for (int per_log2 = 0; per_log2 <= 6; ++per_log2) {
        if (per_log2 == 5) continue;
        for (int variant = 0; variant < 4; ++variant)
            for (int mode = 0; mode < 3; ++mode) {
                const int gn_log2 = 1 + variant % 2 < per_log2 ? 1 + variant % 2 : per_log2;
                const bool regroup = variant >= 2;
                for (int m = 1; m <= 40; ++m)
                    for (int n = 1; n <= 40; ++n, ++cases)
                        if (int e = check(m, n, gn_log2, mode, regroup, per_log2)) return std::printf("tiles %d x %d, %d places, columns per group %d, regrouped %d, mode %d: check %d failed\n", m, n, 1 << per_log2, 1 << gn_log2, regroup, mode, e), 1;
                const int small[][2] = {{4, 80}, {2, 120}, {256, 2}, {128, 4}, {1, 512}, {512, 1}, {3, 170}};
                for (auto &b : small) {
                    ++cases;
                    if (int e = check(b[0], b[1], gn_log2, mode, regroup, per_log2)) return std::printf("tiles %d x %d, %d places, columns per group %d, regrouped %d, mode %d: check %d failed\n", b[0], b[1], 1 << per_log2, 1 << gn_log2, regroup, mode, e), 1;
                }
            }
    }
    std::printf("ok %ld\n", cases);
    return 0;
}
