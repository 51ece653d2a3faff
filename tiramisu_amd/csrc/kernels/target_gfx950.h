// The machine that the emitters and kernels of this back-end are shaped for: one MI355X (gfx950).
// Plain constants and the tile model, usable from host C++ (the recognisers, the runtime's dispatch)
// and from device code alike; nothing else in the tree spells these numbers.
#ifndef TIRAMISU_AMD_TARGET_GFX950_H
#define TIRAMISU_AMD_TARGET_GFX950_H

namespace ttarget {

constexpr int COMPUTE_UNITS = 256;        // 8 XCDs x 32
constexpr int XCDS = 8;                   // each with its own L2; workgroup ids are dealt to them round-robin
constexpr int WAVEFRONT = 64;
constexpr int LDS_BYTES_PER_CU = 160 * 1024;
constexpr int MAX_THREADS_PER_WORKGROUP = 1024;

// Square C tiles of the fp32 MFMA kernel and the share of the matrix-core rate that a tile of each size
// sustains (larger tiles re-read less through LDS); 256 and 192 are used for whole tiles only.
struct square_tile { int edge; double rate; bool whole_only; };
constexpr square_tile SQUARE_TILES[] = {{256, 1.0, true}, {192, 0.9, true}, {128, 0.8, false}, {64, 0.68, false}};

// The square tile whose launch is modelled fastest for an M x N result: a compute unit works through
// ceil(tiles / COMPUTE_UNITS) tiles, each costing its area over its rate.
inline int square_tile_for(long M, long N) {
    double best = 0;
    int edge = 64;
    for (const square_tile &c : SQUARE_TILES) {
        if (c.whole_only && (M % c.edge != 0 || N % c.edge != 0)) continue;
        if (c.edge == 128 && M < 128) continue;
        const long tiles = ((M + c.edge - 1) / c.edge) * ((N + c.edge - 1) / c.edge);
        const double cost = (double)((tiles + COMPUTE_UNITS - 1) / COMPUTE_UNITS) * c.edge * c.edge / c.rate;
        if (best == 0 || cost < best) { best = cost; edge = c.edge; }
    }
    return edge;
}

}  // namespace ttarget
#endif
