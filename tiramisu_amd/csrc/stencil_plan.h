// How the stencil emitter cuts a time loop into launches and a launch into workgroups: plain integer arithmetic,
// shared by the emitter (recognize.cpp), which prints the result as the macros of kernels/stencil2d_regs.hip.h, and by
// the host-side model of that kernel's loads and stores (tests/programs/stencil_address_model.cpp).
#ifndef TIRAMISU_AMD_STENCIL_PLAN_H
#define TIRAMISU_AMD_STENCIL_PLAN_H
#include <algorithm>
#include <vector>

namespace tstencil {

constexpr int REGION_COLUMNS = 256;   // a staged region is one wavefront wide: 64 lanes x 4 columns

// A launch: `steps` time steps from step `first` on, in kernel mode `mode` (0 between the two planes, 1 into a third
// plane, 2 from the third plane into both planes, 3 a single step out of place).
struct chunk { long first; int steps; int mode; };

// Most steps that one launch may fuse: at least half of the staged rows and columns must remain as the tile.
inline int step_cap(int wanted, int radius, int region_rows) {
    int rcap = wanted;
    while (rcap > 1 && (4 * rcap * radius > region_rows || 4 * ((rcap * radius + 3) / 4 * 4) > REGION_COLUMNS)) rcap -= 1;
    return rcap < 1 ? 1 : rcap;
}

// On return both planes must hold exactly what the un-tiled loop leaves there: the last step in one, the last but one
// in the other.  A launch between the two planes advances an odd number of steps.
//  * With a third plane: odd chunks between the planes, the last of them into the third plane, and a final launch
//    that reads the third plane and writes both planes (the values of its last step but one and of its last step), so
//    no launch is spent on a single step.
//  * Without (fewer than 3 steps, or no third plane wanted): odd chunks for all steps but the last, then the last alone.
//  * `planar`: one step out of place.
inline std::vector<chunk> plan_time_loop(long first_step, long steps, int rcap, bool planar, bool temp_plane) {
    const int rmax = rcap % 2 == 0 ? rcap - 1 : rcap;
    if (rcap < 2) temp_plane = false;     // the launch that leaves the third plane advances two steps or more
    auto odd_chunks = [&](long first, long count) {
        std::vector<chunk> out;
        while (count > 0) {
            int c = (int)std::min<long>(rmax, count);
            if (c % 2 == 0) c -= 1;
            out.push_back({first, c, 0});
            first += c;
            count -= c;
        }
        return out;
    };
    std::vector<chunk> chunks;
    if (planar) {
        chunks.push_back({first_step, 1, 3});
    } else if (temp_plane) {
        // the final launch's length: the one that needs the fewest launches (the longest of those)
        int best = 2;
        size_t best_n = 0;
        for (int fin = (int)std::min<long>(rcap, steps - 1); fin >= 2; fin--) {
            const size_t n = odd_chunks(first_step, steps - fin).size();
            if (best_n == 0 || n < best_n) { best = fin; best_n = n; }
        }
        chunks = odd_chunks(first_step, steps - best);
        chunks.back().mode = 1;
        chunks.push_back({first_step + steps - best, best, 2});
    } else {
        chunks = odd_chunks(first_step, steps - 1);
        chunks.push_back({first_step + steps - 1, 1, 0});
    }
    return chunks;
}

// The tiles of one launch over a plane of NY x NX cells whose iteration domain is rows y0..y1, columns x0..x1.
struct launch_geometry {
    int halo_rows, halo_columns;      // steps x radius, the columns rounded up to a multiple of 4
    int tile_rows, tile_columns;      // what a workgroup writes: region minus the halo on both sides
    long tiles_x, tiles_y;
    long ibx0, ibx1, iby0, iby1;      // inclusive ranges of the tiles whose staged region lies inside the iteration domain
    long interior, edge_tiles;
    int rows_edge;                    // rows per thread of a boundary slice
    int slice_rows, slices;           // rows a boundary slice writes, slices per boundary tile
};

inline launch_geometry plan_launch(long NY, long NX, long y0, long y1, long x0, long x1, int radius, int steps, int waves, int rows) {
    auto ceil_div = [](long a, long b) { return a >= 0 ? (a + b - 1) / b : -((-a) / b); };
    auto floor_div = [](long a, long b) { return a >= 0 ? a / b : -((-a + b - 1) / b); };
    launch_geometry g;
    const int LH = waves * rows, LW = REGION_COLUMNS;
    g.halo_rows = steps * radius;
    g.halo_columns = (steps * radius + 3) / 4 * 4;
    g.tile_rows = LH - 2 * g.halo_rows;
    g.tile_columns = LW - 2 * g.halo_columns;
    g.tiles_x = (NX + g.tile_columns - 1) / g.tile_columns;
    g.tiles_y = (NY + g.tile_rows - 1) / g.tile_rows;
    // tiles whose staged region [b*T - H, b*T - H + L) lies inside the iteration domain
    g.ibx0 = std::max<long>(0, ceil_div(x0 + g.halo_columns, g.tile_columns));
    g.ibx1 = std::min<long>(g.tiles_x - 1, floor_div(x1 - LW + 1 + g.halo_columns, g.tile_columns));
    g.iby0 = std::max<long>(0, ceil_div(y0 + g.halo_rows, g.tile_rows));
    g.iby1 = std::min<long>(g.tiles_y - 1, floor_div(y1 - LH + 1 + g.halo_rows, g.tile_rows));
    if (g.ibx0 > g.ibx1 || g.iby0 > g.iby1) { g.iby0 = g.tiles_y; g.iby1 = g.tiles_y - 1; g.ibx0 = 0; g.ibx1 = g.tiles_x - 1; }   // no interior tile
    g.interior = (g.ibx1 - g.ibx0 + 1) * (g.iby1 - g.iby0 + 1);
    g.edge_tiles = g.tiles_x * g.tiles_y - g.interior;
    // boundary tiles are cut into slices of half the rows per thread when the halo allows it
    g.rows_edge = rows / 2;
    if (g.rows_edge < radius || g.rows_edge < 1 || waves * g.rows_edge - 2 * g.halo_rows < 8) g.rows_edge = rows;
    g.slice_rows = waves * g.rows_edge - 2 * g.halo_rows;
    g.slices = (g.tile_rows + g.slice_rows - 1) / g.slice_rows;
    return g;
}

}  // namespace tstencil
#endif
