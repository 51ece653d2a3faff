// Time-tiled 2-D stencil sweep for gfx950: ST_R consecutive time steps of
//     new(y, x) = ST_EXPR( old(y+dy, x+dx) ... )   for (y, x) in the iteration domain,
// on a ping-pong pair of planes, with one global read and one global write per cell for all
// ST_R steps.  The stencil stays on the vector ALUs; LDS holds the tile with its halo.
//
// Each workgroup owns an ST_TH x ST_TW tile of the plane.  It stages the tile plus a halo of
// ST_R*ST_RAD rows (and the same number of columns, rounded up to 4 so that rows stay 16-byte
// aligned) in LDS, advances the staged region ST_R steps in place -- every step the region
// that still holds correct values shrinks by ST_RAD on each side -- and writes the tile's
// centre to the other plane.  Work is dealt in "quads" (4 consecutive cells of a row, one
// 16-byte LDS/global access); a thread keeps the same quads through load, all steps and store.
//
// Cells outside the iteration domain (the fixed boundary) are never written.  When a step
// needs their value it takes the one their plane holds: both planes' values are fetched at
// load time, so the two planes may hold different boundary values, exactly as in the
// un-tiled program.  Reading plane `src` and writing plane `1-src` requires ST_R to be odd;
// the host code composes the time loop from odd chunks.
//
// Macros supplied by the emitter before this file is included:
//   ST_NAME            kernel name
//   ST_NY, ST_NX       plane extents (rows, columns)
//   ST_Y0, ST_Y1, ST_X0, ST_X1   inclusive bounds of the iteration domain
//   ST_TH, ST_TW       tile extents; ST_TW % 4 == 0
//   ST_R               time steps fused in one launch (odd)
//   ST_RAD             stencil radius
//   ST_NT              threads per workgroup
//   ST_EXPR            expression of the new value in terms of ST_AT(dy, dx)
#include <hip/hip_runtime.h>
#include <stdint.h>

#define ST_HY (ST_R * ST_RAD)                       /* halo rows */
#define ST_HX ((ST_R * ST_RAD + 3) / 4 * 4)         /* halo columns, multiple of 4 */
#define ST_LH (ST_TH + 2 * ST_HY)
#define ST_LW (ST_TW + 2 * ST_HX)
#define ST_QPR (ST_LW / 4)                          /* quads per staged row */
#define ST_NQ (ST_LH * ST_QPR)                      /* quads in the staged region */
#define ST_QPT ((ST_NQ + ST_NT - 1) / ST_NT)        /* quads per thread */
#define ST_PAD 4                                    /* floats before/after the region in LDS */

typedef float st_f4 __attribute__((ext_vector_type(4)));

extern "C" __global__ void __launch_bounds__(ST_NT)
ST_NAME(float *__restrict__ planes, const int src_plane)
{
    __shared__ __attribute__((aligned(16))) float lds_raw[ST_LH * ST_LW + 2 * ST_PAD];
    float *L = lds_raw + ST_PAD;
    const float *__restrict__ src = planes + (size_t)src_plane * ST_NY * ST_NX;
    float *__restrict__ dst = planes + (size_t)(1 - src_plane) * ST_NY * ST_NX;
    const int ty0 = blockIdx.y * ST_TH - ST_HY;     // plane row of staged row 0
    const int tx0 = blockIdx.x * ST_TW - ST_HX;     // plane column of staged column 0
    const int tid = threadIdx.x;

    st_f4 keep_src[ST_QPT], keep_dst[ST_QPT];       // boundary values of both planes
    // ---- stage the region
#pragma unroll
    for (int k = 0; k < ST_QPT; k++) {
        const int q = tid + k * ST_NT;
        st_f4 v = {0.f, 0.f, 0.f, 0.f}, o = {0.f, 0.f, 0.f, 0.f};
        if (q < ST_NQ) {
            const int row = q / ST_QPR, col = (q % ST_QPR) * 4;
            const int gy = ty0 + row, gx = tx0 + col;
            if (gy >= 0 && gy < ST_NY) {
                const bool all_in = (ST_NX % 4 == 0) && gx >= 0 && gx + 3 < ST_NX;
                const bool interior = gy >= ST_Y0 && gy <= ST_Y1 && gx >= ST_X0 && gx + 3 <= ST_X1;
                if (all_in) {
                    v = *reinterpret_cast<const st_f4 *>(src + (size_t)gy * ST_NX + gx);
                    if (!interior) o = *reinterpret_cast<const st_f4 *>(dst + (size_t)gy * ST_NX + gx);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                    {
                        // rows whose length is not a multiple of 4: element loads from a clamped
                        // (always valid) column, the value selected afterwards
                        const int xx = gx + e;
                        const bool inp = xx >= 0 && xx < ST_NX;
                        const size_t at = (size_t)gy * ST_NX + (inp ? xx : 0);
                        const float a = src[at], b = dst[at];
                        v[e] = inp ? a : 0.f;
                        o[e] = inp ? b : 0.f;
                    }
                }
            }
            *reinterpret_cast<st_f4 *>(L + row * ST_LW + col) = v;
        }
        keep_src[k] = v;
        keep_dst[k] = o;
    }
    __syncthreads();

    // ---- ST_R steps in place
#pragma unroll
    for (int s = 1; s <= ST_R; s++) {
        st_f4 nv[ST_QPT];
#pragma unroll
        for (int k = 0; k < ST_QPT; k++) {
            const int q = tid + k * ST_NT;
            const int row = q / ST_QPR, col = (q % ST_QPR) * 4;
            nv[k] = keep_src[k];
            // rows that still have all their neighbours at this step
            if (q < ST_NQ && row >= s * ST_RAD && row < ST_LH - s * ST_RAD) {
                const int gy = ty0 + row, gx = tx0 + col;
                // window of old values around the quad: rows -RAD..RAD, columns -RAD..3+RAD
                float w[2 * ST_RAD + 1][4 + 2 * ST_RAD];
#pragma unroll
                for (int dy = -ST_RAD; dy <= ST_RAD; dy++) {
                    const float *p = L + (row + dy) * ST_LW + col;
                    const st_f4 c = *reinterpret_cast<const st_f4 *>(p);
#pragma unroll
                    for (int e = 0; e < 4; e++) w[dy + ST_RAD][e + ST_RAD] = c[e];
#pragma unroll
                    for (int e = 1; e <= ST_RAD; e++) {
                        w[dy + ST_RAD][ST_RAD - e] = p[-e];
                        w[dy + ST_RAD][3 + ST_RAD + e] = p[3 + e];
                    }
                }
                const bool row_in = gy >= ST_Y0 && gy <= ST_Y1;
#pragma unroll
                for (int e = 0; e < 4; e++) {
#define ST_AT(dy, dx) w[(dy) + ST_RAD][e + (dx) + ST_RAD]
                    const float computed = (ST_EXPR);
#undef ST_AT
                    const bool in_dom = row_in && gx + e >= ST_X0 && gx + e <= ST_X1;
                    // a fixed cell shows the value of the plane that step s lives in
                    nv[k][e] = in_dom ? computed : ((s & 1) ? keep_dst[k][e] : keep_src[k][e]);
#ifdef ST_DEBUG_HOOK
                    ST_DEBUG_HOOK(s, k, e, row, col, gy, gx, in_dom, computed)
#endif
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < ST_QPT; k++) {
            const int q = tid + k * ST_NT;
            const int row = q / ST_QPR, col = (q % ST_QPR) * 4;
            if (q < ST_NQ && row >= s * ST_RAD && row < ST_LH - s * ST_RAD) {
                *reinterpret_cast<st_f4 *>(L + row * ST_LW + col) = nv[k];
                if (s == ST_R) {
                    // ---- write the tile centre (cells of the domain only)
                    const int gy = ty0 + row, gx = tx0 + col;
                    if (row >= ST_HY && row < ST_HY + ST_TH && col >= ST_HX && col < ST_HX + ST_TW &&
                        gy >= ST_Y0 && gy <= ST_Y1) {
                        if ((ST_NX % 4 == 0) && gx >= ST_X0 && gx + 3 <= ST_X1) {
                            *reinterpret_cast<st_f4 *>(dst + (size_t)gy * ST_NX + gx) = nv[k];
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                if (gx + e >= ST_X0 && gx + e <= ST_X1) dst[(size_t)gy * ST_NX + gx + e] = nv[k][e];
                        }
                    }
                }
            }
        }
        if (s < ST_R) __syncthreads();
    }
}

#undef ST_HY
#undef ST_HX
#undef ST_LH
#undef ST_LW
#undef ST_QPR
#undef ST_NQ
#undef ST_QPT
#undef ST_PAD
