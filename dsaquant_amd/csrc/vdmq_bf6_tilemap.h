// Tile order of the bf6 GEMM kernels (vdmq_bf6.hip): which output tile the workgroup at a CU position of an XCD takes
// in each round.  Plain C++ with no device types, so that the host launcher, both kernels and a host-compiled checker
// share one definition.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define VDMQ_TILEMAP_FN __host__ __device__ inline
#else
#define VDMQ_TILEMAP_FN inline
#endif

namespace vdmq {

constexpr int kBf6Xcds = 8;

// The tiles_m x tiles_n grid of output tiles is cut into super-tiles of `per` = 1 << per_log2 places, one per CU of
// an XCD, so that the XCD's CUs work on neighbouring tiles at the same time and share their operand rows in its L2:
//
//   main region   the full groups of gm = per / gn rows and gn = 1 << group_n_log2 columns, n fastest;
//   right edge    the tiles_n % gn columns left over, beside the main region's rows, as super-tiles of edge_n_rows
//                 rows x those columns;
//   bottom edge   the tiles_m % gm rows left over, all columns, as super-tiles of those rows x edge_m_cols columns.
//
// Edge super-tiles either keep the main shape's rows (columns) and are partly empty, or are regrouped: more rows
// (columns) so that the places are filled.  A workgroup that keeps its place in every super-tile of its XCD spends a
// round on each, however full, so the regrouped edges save rounds on large problems; on small ones the partly empty
// super-tiles spread the few tiles over more XCDs.
//
// The sequence is main, right edge, bottom edge.  XCD x takes either every eighth super-tile (x, x + 8, ...) or, with
// `contig`, the run [start[x], start[x + 1]).
struct Bf6TileMap {
    int tiles_m, tiles_n;
    int per_log2, group_n_log2;
    int main_n, n_main;            /* full super-tile columns; super-tiles of the main region */
    int edge_n_cols, edge_n_rows, n_edge_n;
    int edge_m_rows, edge_m_cols, n_edge_m;
    int total_super;
    int contig;
    int start[kBf6Xcds + 1];
};

// Shape part of the map (everything but contig / start) for the main shape (per >> gn_log2) x (1 << gn_log2).
// A regrouped edge super-tile has at most 16 rows (columns) of tiles however few columns (rows) are left: beyond that
// its operand rows no longer fit what an XCD's L2 turns over in a K step.
VDMQ_TILEMAP_FN void bf6_tilemap_shape(Bf6TileMap &tm, int tiles_m, int tiles_n, int per_log2, int gn_log2, bool regroup) {
    const int per = 1 << per_log2, gn = 1 << gn_log2, gm = per >> gn_log2;
    tm.tiles_m = tiles_m;
    tm.tiles_n = tiles_n;
    tm.per_log2 = per_log2;
    tm.group_n_log2 = gn_log2;
    tm.main_n = tiles_n / gn;
    const int main_m = tiles_m / gm;
    tm.n_main = main_m * tm.main_n;
    tm.edge_n_cols = tiles_n - tm.main_n * gn;
    tm.edge_n_rows = tm.edge_n_cols == 0 ? 1 : !regroup ? gm : (per / tm.edge_n_cols < 16 ? per / tm.edge_n_cols : 16);
    tm.n_edge_n = tm.edge_n_cols == 0 ? 0 : (main_m * gm + tm.edge_n_rows - 1) / tm.edge_n_rows;
    tm.edge_m_rows = tiles_m - main_m * gm;
    tm.edge_m_cols = tm.edge_m_rows == 0 ? 1 : !regroup ? gn : (per / tm.edge_m_rows < 16 ? per / tm.edge_m_rows : 16);
    tm.n_edge_m = tm.edge_m_rows == 0 ? 0 : (tiles_n + tm.edge_m_cols - 1) / tm.edge_m_cols;
    tm.total_super = tm.n_main + tm.n_edge_n + tm.n_edge_m;
}

// The tile at `place` (0 ... per - 1) of super-tile st; false: that place is empty.
VDMQ_TILEMAP_FN bool bf6_tilemap_locate(const Bf6TileMap &tm, int st, int place, int &tile_m, int &tile_n) {
    const int gn_log2 = tm.group_n_log2, gm_log2 = tm.per_log2 - gn_log2;
    if (st < tm.n_main) {
        const int r = st / tm.main_n, c = st - r * tm.main_n;
        tile_m = (r << gm_log2) + (place >> gn_log2);
        tile_n = (c << gn_log2) + (place & ((1 << gn_log2) - 1));
        return true;
    }
    const int rows_main = (tm.tiles_m >> gm_log2) << gm_log2;
    st -= tm.n_main;
    if (st < tm.n_edge_n) {
        const int pr = place / tm.edge_n_cols;
        tile_m = st * tm.edge_n_rows + pr;
        tile_n = (tm.main_n << gn_log2) + place - pr * tm.edge_n_cols;
        return pr < tm.edge_n_rows && tile_m < rows_main;
    }
    st -= tm.n_edge_n;
    const int pr = place / tm.edge_m_cols;
    tile_m = rows_main + pr;
    tile_n = st * tm.edge_m_cols + place - pr * tm.edge_m_cols;
    return pr < tm.edge_m_rows && tile_n < tm.tiles_n;
}

// Tiles in the super-tiles [0, st) of the sequence.
VDMQ_TILEMAP_FN int64_t bf6_tilemap_tiles_before(const Bf6TileMap &tm, int64_t st) {
    const int gm_log2 = tm.per_log2 - tm.group_n_log2;
    const int64_t rows_main = (tm.tiles_m >> gm_log2) << gm_log2;
    if (st <= tm.n_main) return st << tm.per_log2;
    int64_t tiles = static_cast<int64_t>(tm.n_main) << tm.per_log2;
    st -= tm.n_main;
    if (st <= tm.n_edge_n) {
        const int64_t rows = st * tm.edge_n_rows < rows_main ? st * tm.edge_n_rows : rows_main;
        return tiles + rows * tm.edge_n_cols;
    }
    tiles += rows_main * tm.edge_n_cols;
    st -= tm.n_edge_n;
    const int64_t cols = st * tm.edge_m_cols < tm.tiles_n ? st * tm.edge_m_cols : tm.tiles_n;
    return tiles + cols * tm.edge_m_rows;
}

// Super-tile of XCD `xcd` in its round `seq`, or -1 when its share is done.
VDMQ_TILEMAP_FN int bf6_tilemap_super(const Bf6TileMap &tm, int xcd, int seq) {
    const int st = tm.contig ? tm.start[xcd] + seq : seq * kBf6Xcds + xcd;
    return st < (tm.contig ? tm.start[xcd + 1] : tm.total_super) ? st : -1;
}

// Contiguous runs: cut the sequence so that the XCDs get equal numbers of tiles (`by_tiles`: a CU is refilled as
// soon as it is free, time goes with the tiles) or of super-tiles (a workgroup that keeps its place in every
// super-tile of its XCD spends a round per super-tile, full or not).  Returns the longest run.
VDMQ_TILEMAP_FN int bf6_tilemap_runs(Bf6TileMap &tm, bool by_tiles) {
    const int64_t all_tiles = static_cast<int64_t>(tm.tiles_m) * tm.tiles_n;
    tm.contig = 1;
    tm.start[0] = 0;
    int longest = 0;
    for (int x = 1; x <= kBf6Xcds; ++x) {
        int64_t lo = tm.start[x - 1], hi = tm.total_super;
        if (by_tiles) {
            const int64_t want = (all_tiles * x + kBf6Xcds - 1) / kBf6Xcds;
            while (lo < hi) {
                const int64_t mid = (lo + hi) / 2;
                if (bf6_tilemap_tiles_before(tm, mid) >= want) hi = mid; else lo = mid + 1;
            }
        } else {
            lo = (static_cast<int64_t>(tm.total_super) * x + kBf6Xcds - 1) / kBf6Xcds;
        }
        tm.start[x] = x == kBf6Xcds ? tm.total_super : static_cast<int>(lo);
        if (tm.start[x] - tm.start[x - 1] > longest) longest = tm.start[x] - tm.start[x - 1];
    }
    return longest;
}

}  // namespace vdmq
