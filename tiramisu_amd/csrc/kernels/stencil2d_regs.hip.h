// Time-tiled 2-D stencil sweep for gfx950 with the tile held in registers: ST_R consecutive
// time steps of
//     new(y, x) = ST_EXPR( old(y+dy, x+dx) ... )   for (y, x) in the iteration domain,
// on a ping-pong pair of planes, with one global read and one global write per cell for all
// ST_R steps.  The stencil stays on the vector ALUs.
//
// A workgroup of ST_W wavefronts stages a region of ST_W*ST_RPT rows by 256 columns: wavefront w
// owns rows [w*ST_RPT, (w+1)*ST_RPT), lane l owns columns [4l, 4l+4) of each of them, so a thread
// keeps a strip of ST_RPT quads in registers through load, all steps and store.
//   * horizontal neighbours live in the adjacent lanes of the same wavefront and arrive through
//     DPP wavefront shifts (no memory traffic); the region is exactly one wavefront wide, so no
//     value ever crosses a wavefront horizontally;
//   * vertical neighbours across the strip boundary live in the wavefront above / below: every
//     step each wavefront publishes its ST_RAD top and bottom rows in LDS (double-buffered by the
//     step's parity, one barrier per step) and reads its neighbours' rows.
// Every step the part of the region that still holds correct values shrinks by ST_RAD on each
// side; after ST_R steps the centre (ST_TH x ST_TW) is written to the other plane.  Values outside
// the shrinking valid part are computed from stale data and never used.
//
// Cells outside the iteration domain (the fixed boundary) are never written.  When a step needs
// their value it takes the one their plane holds at that step's parity, so the two planes may hold
// different boundary values, exactly as in the un-tiled program: a thread whose strip contains
// fixed cells keeps the other plane's values of its strip in registers (read once; no launch ever
// writes those cells) and swaps the two values of a fixed cell at every step.  That costs registers
// and checks, so each launch is split in two kernels: ST_NAME for the tiles whose staged region
// lies inside the iteration domain (no checks at all), ST_NAME_EDGE for the others.
//
// Where the values come from and go to (ST_MODE), `p` being the plane that holds the source step:
//   0  read plane p, write plane 1-p (disjoint cells): ST_R must be odd;
//   1  read plane p, write a third plane `temp` that stands in for plane 1-p (ST_R odd), fixed cells included,
//      so that a later launch finds there all it reads;
//   2  read `temp` (standing in for plane p) and write both planes: the values after ST_R - 1 steps to the plane
//      of that step's parity and those after ST_R steps to the other one.  Neither plane is read except for its
//      fixed cells, so ST_R may be even and the time loop can end with a fused launch that leaves both planes
//      exactly as the un-tiled loop does.
//   3  a single step out of place (ST_R = 1): read the first buffer, write another one that comes in the place of
//      `temp`; the fixed cells are the source's and nothing of them is stored.
// The host code composes the time loop from such launches.
//
// Macros supplied by the emitter before this file is included:
//   ST_NAME            kernel name
//   ST_NY, ST_NX       plane extents (rows, columns)
//   ST_Y0, ST_Y1, ST_X0, ST_X1   inclusive bounds of the iteration domain
//   ST_R               time steps fused in one launch
//   ST_MODE            0, 1 or 2: see above
//   ST_RAD             stencil radius (<= 4, <= ST_RPT); 0 for a point-wise map (mode 3): nothing is exchanged
//   ST_W               wavefronts per workgroup
//   ST_RPT             rows per thread
//   ST_RPT_EDGE        rows per thread in the kernel for boundary tiles (a divisor-sized slice
//                      of a tile; launch it with ceil(ST_TH / (ST_W*ST_RPT_EDGE - 2*ST_R*ST_RAD))
//                      workgroups per boundary tile)
//   ST_EXPR            expression of the new value in terms of ST_AT(dy, dx)
//   ST_NAME_EDGE       name of the kernel for the tiles that touch the fixed boundary
//   ST_STREAM          bit 0: staging loads carry the non-temporal hint, bit 1: the stores of the tile centre do
//   ST_GX, ST_GY       number of tiles along x and y
//   ST_IBX0, ST_IBX1, ST_IBY0, ST_IBY1   inclusive ranges of interior tiles (ST_IBY0 = ST_GY and
//                      ST_IBY1 = ST_GY - 1 when there is none); launch ST_NAME with one workgroup
//                      per interior tile and ST_NAME_EDGE with one per remaining tile
// The tile extents follow: ST_TH = ST_W*ST_RPT - 2*ST_R*ST_RAD, ST_TW = 256 - 2*roundup4(ST_R*ST_RAD).
//
// The same text also compiles as plain host C++ (ST_HOST_MODEL defined by the includer, which then supplies
// threadIdx / blockIdx and the few device keywords as stand-ins): every access to global memory goes through the
// ST_GLOBAL_* macros below, the plane geometry may then be run-time values (ST_CONSTEXPR, ST_STATIC_ASSERT), and with
// ST_SKIP_ARITHMETIC the steps are walked without computing -- which leaves exactly the kernel's own loads, stores
// and the conditions they sit under, for a host program to enumerate.
#ifndef ST_HOST_MODEL
#include <hip/hip_runtime.h>
#endif
#include <stdint.h>

#include "target_gfx950.h"

#ifndef ST_CONSTEXPR
#define ST_CONSTEXPR constexpr
#define ST_STATIC_ASSERT(cond, text) static_assert(cond, text)
#define ST_SKIP_ARITHMETIC 0
// p: pointer to a quad (16 bytes) or to one cell; stream: ask with the non-temporal hint
#define ST_GLOBAL_LOAD4(p, stream) ((stream) ? __builtin_nontemporal_load(p) : *(p))
#define ST_GLOBAL_LOAD1(p) (*(p))
#define ST_GLOBAL_STORE4(p, v, stream) do { if (stream) __builtin_nontemporal_store((v), (p)); else *(p) = (v); } while (0)
#define ST_GLOBAL_STORE1(p, v) (*(p) = (v))
#endif

#define ST_HY (ST_R * ST_RAD)                       /* halo rows */
#define ST_HX ((ST_R * ST_RAD + 3) / 4 * 4)         /* halo columns, multiple of 4 */
#define ST_LH (ST_W * ST_RPT)
#define ST_LW 256
#define ST_TH (ST_LH - 2 * ST_HY)
#define ST_TW (ST_LW - 2 * ST_HX)
#define ST_CAT2(a, b) a##b
#define ST_CAT(a, b) ST_CAT2(a, b)

// The planes of a launch.  Plane src_plane holds (or `temp` stands in for) the source step; after ST_R steps the
// values belong in plane (src_plane + ST_R) % 2.
#define ST_PLANE(p) (planes + (size_t)(p) * ST_NY * ST_NX)
#define ST_PLANES                                                                                              \
    const float *__restrict__ src = ST_MODE == 2 ? temp : ST_PLANE(src_plane);                                 \
    float *__restrict__ dst = (ST_MODE == 1 || ST_MODE == 3) ? temp : ST_PLANE((src_plane + ST_R) & 1);        \
    float *__restrict__ dst_prev = ST_MODE == 2 ? ST_PLANE((src_plane + ST_R - 1) & 1) : nullptr;              \
    const float *fixed_other = ST_PLANE(ST_MODE == 3 ? src_plane : 1 - src_plane);

#ifndef TIRAMISU_AMD_STENCIL2D_REGS_COMMON
#define TIRAMISU_AMD_STENCIL2D_REGS_COMMON
#ifdef ST_HOST_MODEL
typedef float st_f4 __attribute__((vector_size(16)));
#else
typedef float st_f4 __attribute__((ext_vector_type(4)));
#endif

// lane i receives lane i-1's value; lane 0, which has no such neighbour, reads 0 (its cells next to the region's
// edge are stale from the first step on and never written).  With nothing to keep for the lanes out of range, the
// compiler folds the shift into the add that consumes it (v_add_f32_dpp) instead of issuing a move.
__device__ __forceinline__ float st_from_left(float v) {
    const int i = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, i, 0x138 /* wave_shr:1 */, 0xf, 0xf, true));
}
// lane i receives lane i+1's value; lane 63 reads 0
__device__ __forceinline__ float st_from_right(float v) {
    const int i = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, i, 0x130 /* wave_shl:1 */, 0xf, 0xf, true));
}

// Four cells of row gy starting at column gx (a multiple of 4) of a plane of NY x NX cells;
// cells outside the plane read as 0.  With CHECK false the quad is known to be inside.
// Element loads always use a clamped (valid) address and select afterwards.  `plane` carries no
// restrict qualifier: the boundary path reads the plane that the same kernel later writes.
// STREAM: the quad is asked for with the non-temporal hint (read once by this launch: it should not displace the
// halo rows and columns that neighbouring tiles share in the L2).  NY, NX are compile-time constants in a kernel.
template <bool CHECK, bool STREAM = false>
__device__ __forceinline__ st_f4 st_load_quad(const float *plane, int gy, int gx, const int NY, const int NX) {
    st_f4 v = {0.f, 0.f, 0.f, 0.f};
    if (NX % 4 == 0) {
        if (!CHECK) return ST_GLOBAL_LOAD4(reinterpret_cast<const st_f4 *>(plane + (size_t)gy * NX + gx), STREAM);
        const bool in = gy >= 0 && gy < NY && gx >= 0 && gx < NX;
        const st_f4 a = ST_GLOBAL_LOAD4(reinterpret_cast<const st_f4 *>(plane + (in ? (size_t)gy * NX + gx : (size_t)0)), false);
        return in ? a : v;
    }
    const bool row_in = !CHECK || (gy >= 0 && gy < NY);
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int xx = gx + e;
        const bool in = row_in && (!CHECK || (xx >= 0 && xx < NX));
        const float a = ST_GLOBAL_LOAD1(plane + (in ? (size_t)gy * NX + xx : (size_t)0));
        v[e] = in ? a : 0.f;
    }
    return v;
}
#endif

// One workgroup advances the region of ST_W*RPT rows whose centre starts at plane row `oy`, column
// `ox`, and writes the centre rows below `row_end`.
// `fixed_other`: the plane whose fixed cells show at the steps of the other parity than the source's; `dst_prev`:
// where the values of the last step but one go (mode 2 only).
template <bool EDGE, int RPT>
__device__ __forceinline__ void ST_CAT(ST_NAME, _sweep)(const float *__restrict__ src, float *__restrict__ dst, float *__restrict__ dst_prev,
                                                        const float *fixed_other, st_f4 *xch, int oy, int ox, int row_end) {
    // values stay in registers from one step to the next: without this the multiply that ends a
    // step would be fused with an add of the next one, and results would differ from the
    // un-tiled program's
#pragma clang fp contract(off)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    ST_CONSTEXPR int CENTRE_ROWS = ST_W * RPT - 2 * ST_HY;
    ST_STATIC_ASSERT(CENTRE_ROWS > 0 && RPT >= ST_RAD, "the halo leaves no rows to write");
    const int gy0 = oy - ST_HY + wave * RPT;              // plane row of my first row
    const int gx = ox - ST_HX + 4 * lane;                 // plane column of my quads
    const int wave_up = wave > 0 ? wave - 1 : 0, wave_dn = wave < ST_W - 1 ? wave + 1 : ST_W - 1;

    st_f4 cur[RPT], other[EDGE ? RPT : 1];   // other: the other plane's values (fixed cells only)
#pragma unroll
    for (int r = 0; r < RPT; r++) {
        cur[r] = st_load_quad<EDGE, (ST_STREAM & 1) != 0>(src, gy0 + r, gx, ST_NY, ST_NX);
        if (EDGE) other[r] = st_load_quad<true>(fixed_other, gy0 + r, gx, ST_NY, ST_NX);
    }

    // xch[parity][wave][top|bottom][row][lane]
    auto slot = [&](int parity, int w, int side, int i) -> st_f4 * {
        return xch + ((((parity * ST_W + w) * 2 + side) * ST_RAD + i) * 64 + lane);
    };

    // ---- write the tile centre: the cells of the domain, or in mode 1 all cells of the plane (a fixed cell then
    // holds the value of the plane that `to` stands in for)
    ST_CONSTEXPR int WY0 = ST_MODE == 1 ? 0 : ST_Y0, WY1 = ST_MODE == 1 ? ST_NY - 1 : ST_Y1;
    ST_CONSTEXPR int WX0 = ST_MODE == 1 ? 0 : ST_X0, WX1 = ST_MODE == 1 ? ST_NX - 1 : ST_X1;
    auto store_centre = [&](float *__restrict__ to) {
        if (4 * lane >= ST_HX && 4 * lane < ST_HX + ST_TW) {
#pragma unroll
            for (int r = 0; r < RPT; r++) {
                const int row = wave * RPT + r, gy = gy0 + r;
                if (row < ST_HY || row >= ST_HY + CENTRE_ROWS || gy >= row_end) continue;
                if (EDGE && (gy < WY0 || gy > WY1)) continue;
                if ((ST_NX % 4 == 0) && (!EDGE || (gx >= WX0 && gx + 3 <= WX1))) {
                    ST_GLOBAL_STORE4(reinterpret_cast<st_f4 *>(to + (size_t)gy * ST_NX + gx), cur[r], (ST_STREAM & 2) != 0);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (!EDGE || (gx + e >= WX0 && gx + e <= WX1)) ST_GLOBAL_STORE1(to + (size_t)gy * ST_NX + gx + e, cur[r][e]);
                }
            }
        }
    };

#pragma unroll
    for (int s = 1; s <= ST_R; s++) {
        const int parity = s & 1;
        if (ST_MODE == 2 && s == ST_R) store_centre(dst_prev);   // the values after ST_R - 1 steps
        if (ST_SKIP_ARITHMETIC) continue;
#pragma unroll
        for (int i = 0; i < ST_RAD; i++) {
            *slot(parity, wave, 0, i) = cur[i];
            *slot(parity, wave, 1, i) = cur[RPT - ST_RAD + i];
        }
        if (ST_RAD > 0) __syncthreads();
        // my rows with ST_RAD rows of the neighbouring wavefronts above and below
        st_f4 ext[RPT + 2 * ST_RAD];
#pragma unroll
        for (int i = 0; i < ST_RAD; i++) {
            ext[i] = *slot(parity, wave_up, 1, i);
            ext[ST_RAD + RPT + i] = *slot(parity, wave_dn, 0, i);
        }
#pragma unroll
        for (int r = 0; r < RPT; r++) ext[ST_RAD + r] = cur[r];
#pragma unroll
        for (int r = 0; r < RPT; r++) {
            // Old value at row r + dy, column e + dx of the quad (columns -RAD .. 3 + RAD): columns outside the quad
            // come from the adjacent lane.  The shift is written where the value is used, once per use: the compiler
            // folds a lane shift into the add that consumes it (v_add_f32_dpp) only when the two are a few
            // instructions apart, and a shift folded that way costs no instruction.
            auto old_at = [&](int dy, int col) -> float {
                const st_f4 &row = ext[r + ST_RAD + dy];
                return col < 0 ? st_from_left(row[4 + col]) : col > 3 ? st_from_right(row[col - 4]) : row[col];
            };
            const bool row_in = !EDGE || (gy0 + r >= ST_Y0 && gy0 + r <= ST_Y1);
#pragma unroll
            for (int e = 0; e < 4; e++) {
#define ST_AT(dy, dx) old_at((dy), e + (dx))
                const float computed = (ST_EXPR);
#undef ST_AT
                if (EDGE) {
                    // a fixed cell shows the value of the plane that step s lives in: swap
                    const bool in_dom = row_in && gx + e >= ST_X0 && gx + e <= ST_X1;
                    const float before = ext[ST_RAD + r][e], there = other[r][e];
                    cur[r][e] = in_dom ? computed : there;
                    other[r][e] = in_dom ? there : before;
                } else {
                    cur[r][e] = computed;
                }
            }
        }
    }

    store_centre(dst);
}

// The tiles outside the interior rectangle, in the order: full tile rows above the interior
// rectangle, full rows below it, then the tiles left and right of it row by row.  These tiles are
// few (one ring), so each is cut into ST_EDGE_SUB horizontal slices of ST_W*ST_RPT_EDGE staged
// rows, one workgroup each: more and lighter workgroups (the swap registers come on top of the
// strip) instead of one heavy workgroup per tile.  eb is the index of the slice.
#define ST_TH_EDGE (ST_W * ST_RPT_EDGE - 2 * ST_HY)
#define ST_EDGE_SUB ((ST_TH + ST_TH_EDGE - 1) / ST_TH_EDGE)
static __device__ __forceinline__ void ST_CAT(ST_NAME, _edge_slice)(const float *__restrict__ src, float *__restrict__ dst,
                                                                     float *__restrict__ dst_prev, const float *fixed_other, st_f4 *xch, int eb)
{
    ST_CONSTEXPR int TOP = ST_IBY0 * ST_GX, BOTTOM = (ST_GY - 1 - ST_IBY1) * ST_GX;
    ST_CONSTEXPR int SIDE = ST_IBX0 + (ST_GX - 1 - ST_IBX1);   // edge tiles per row of the interior band
    const int sub = eb % ST_EDGE_SUB;
    int e = eb / ST_EDGE_SUB, bx, by;
    if (e < TOP) {
        by = e / ST_GX;
        bx = e % ST_GX;
    } else if (e < TOP + BOTTOM) {
        e -= TOP;
        by = ST_IBY1 + 1 + e / ST_GX;
        bx = e % ST_GX;
    } else {
        e -= TOP + BOTTOM;
        const int c = e % (SIDE > 0 ? SIDE : 1);
        by = ST_IBY0 + e / (SIDE > 0 ? SIDE : 1);
        bx = c < ST_IBX0 ? c : ST_IBX1 + 1 + (c - ST_IBX0);
    }
    ST_CAT(ST_NAME, _sweep)<true, ST_RPT_EDGE>(src, dst, dst_prev, fixed_other, xch, by * ST_TH + sub * ST_TH_EDGE, bx * ST_TW, (by + 1) * ST_TH);
}

// Interior tiles: one workgroup per tile of the rectangle [ST_IBX0, ST_IBX1] x [ST_IBY0, ST_IBY1],
// no bounds checks.  With ST_MERGE the launch carries the edge slices as well, after the ST_NI
// interior workgroups: they are lighter and fill the tail of the launch instead of running as a
// small launch of their own (the edge path needs fewer registers than the interior one, so the
// interior tiles keep their occupancy).
#define ST_NI ((ST_IBY1 >= ST_IBY0 && ST_IBX1 >= ST_IBX0) ? (ST_IBX1 - ST_IBX0 + 1) * (ST_IBY1 - ST_IBY0 + 1) : 0)
extern "C" __global__ void __launch_bounds__(64 * ST_W)
#if ST_OCC > 0
__attribute__((amdgpu_waves_per_eu(ST_OCC)))
#endif
ST_NAME(float *planes, const int src_plane, float *temp)
{
    ST_STATIC_ASSERT(ST_TH > 0 && ST_TW > 0, "the halo leaves no tile: fuse fewer steps or use more rows");
    ST_STATIC_ASSERT(ST_MODE == 2 ? ST_R >= 2 : ST_MODE == 3 ? ST_R == 1 : ST_R % 2 == 1, "a launch between the two planes advances an odd number of steps");
    __shared__ st_f4 xch[2 * ST_W * 2 * (ST_RAD > 0 ? ST_RAD : 1) * 64];
    ST_PLANES
    const int b = blockIdx.x;
#if ST_MERGE
    if (b >= ST_NI) {
        ST_CAT(ST_NAME, _edge_slice)(src, dst, dst_prev, fixed_other, xch, b - ST_NI);
        return;
    }
#endif
    // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2: give every XCD a band
    // of consecutive tiles (row-major), so that tiles running together share their halos in L2.
    ST_CONSTEXPR int IW = ST_IBX1 - ST_IBX0 + 1;
    ST_CONSTEXPR int nb = ST_NI;
#if ST_XCD
    constexpr int XCDS = ttarget::XCDS;
    const int xcd = b % XCDS, per = nb / XCDS, extra = nb % XCDS;
    const int tile = xcd * per + (xcd < extra ? xcd : extra) + b / XCDS;
#else
    const int tile = b;
#endif
    ST_CAT(ST_NAME, _sweep)<false, ST_RPT>(src, dst, dst_prev, fixed_other, xch, (ST_IBY0 + tile / IW) * ST_TH, (ST_IBX0 + tile % IW) * ST_TW, ST_NY);
}

// The edge slices as a launch of their own (used when the launches are not merged).
extern "C" __global__ void __launch_bounds__(64 * ST_W)
ST_NAME_EDGE(float *planes, const int src_plane, float *temp)
{
    __shared__ st_f4 xch[2 * ST_W * 2 * (ST_RAD > 0 ? ST_RAD : 1) * 64];
    ST_PLANES
    ST_CAT(ST_NAME, _edge_slice)(src, dst, dst_prev, fixed_other, xch, blockIdx.x);
}
#undef ST_NI
#undef ST_TH_EDGE
#undef ST_EDGE_SUB

#undef ST_PLANE
#undef ST_PLANES
#undef ST_HY
#undef ST_HX
#undef ST_LH
#undef ST_LW
#undef ST_TH
#undef ST_TW
#undef ST_CAT
#undef ST_CAT2
