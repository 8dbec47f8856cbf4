// What the host decides about a grouped launch, shared by the translation unit that decides (gemm_grouped.hip)
// and the ones that launch (gemm_grouped_<format>.hip through lowbit_gemm_grouped.h).  No kernel code in here.
#pragma once

namespace lowbit {

// Tile sizes of the tall form that workspace sizes depend on (lowbit_gemm_grouped.h checks them against the
// kernel's own constants).
constexpr int G_GN = 256, G_GM_TALL = 256;

// How a grouped launch runs: chosen on the host from the row count, never from the rows per group, which only
// the device knows.
struct GroupedPlan {
    bool tall;      // 256-row tiles (always for the fused gate/up form)
    int splits;     // K splits of the tall form (1 = none)
    int waves;      // waves per workgroup of the tall form: 4 (64 weight rows each) or 8 (32 each, two per SIMD)
    bool one_round; // the launch's workgroups (expected count) all fit the machine at once
};

// Upper bound of the number of `rows`-row tiles: every group adds at most one partly filled tile.
inline int grouped_max_row_tiles(int total_rows, int n_groups, int rows) { return total_rows / rows + n_groups; }

// Column tiles per cell of the tile order (grouped_tile in lowbit_gemm_kernel.h): a whole row of column tiles when
// the launch is a single round of workgroups, else an eighth of it, so that every XCD gets an equal share of
// every row tile.
inline int grouped_chunk(int tiles_n, bool one_round) { return one_round ? tiles_n : (tiles_n + 7) / 8; }

// Workgroups (grid.x) of a grouped launch over at most `row_tiles` row tiles: 8 XCDs x the most cells one of them
// gets x chunk.  Partial tiles of a K split are indexed by workgroup: a workspace holds this many tiles per split.
inline int grouped_grid(int row_tiles, int tiles_n, int chunk) {
    const int cells = row_tiles * ((tiles_n + chunk - 1) / chunk);
    return 8 * ((cells + 7) / 8) * chunk;
}

}  // namespace lowbit
