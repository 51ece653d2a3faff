// Host-side model of the loads and stores of kernels/stencil2d_regs.hip.h.  The kernel header itself is compiled
// here as plain C++ (its ST_HOST_MODEL form): threadIdx / blockIdx are variables of this program, every access to
// global memory lands in the recorders below instead of memory, and the steps are walked without arithmetic.  For
// every plane size, steps per launch, kernel mode and source plane in the sweep, every workgroup and thread of the
// launch that the emitter would make (tiramisu_amd/csrc/stencil_plan.h: the code the emitter itself calls) is run, and
// the program checks that
//   * every load lies inside the buffer it reads, a 16-byte load on a 16-byte boundary, and every cell of the iteration
//     domain is loaded from the launch's source (a launch's source is never one of its destinations: the other plane
//     is read only through the argument that is consulted for fixed cells);
//   * every store lies inside its buffer, and after the launch every cell that the launch owes (the iteration domain;
//     in mode 1 the whole plane) has been written exactly once and no other cell at all;
//   * a whole time loop, cut into launches by the emitter's plan, leaves the last step in the plane of its parity and
//     the last step but one in the other.
// Prints one line per failure and a summary; exit status 0 only when there is none.
// tests/test_stencil_address_model.py compiles and runs it (g++, no GPU, no Tiramisu library).
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../tiramisu_amd/csrc/stencil_plan.h"   // the emitter's own plan

// ---- stand-ins for the device side
struct model_index { unsigned x, y, z; };
static model_index threadIdx, blockIdx;
#define __global__
#define __device__
#define __forceinline__ inline
#define __launch_bounds__(n)
#define __shared__ static
static inline void __syncthreads() {}
static inline int __builtin_amdgcn_update_dpp(int, int v, int, int, int, bool) { return v; }

// ---- the launch under test
struct model_geometry {
    int ny, nx, y0, y1, x0, x1;          // plane and iteration domain
    int gx, gy, ibx0, ibx1, iby0, iby1;  // tiles
    int r, mode;
};
static model_geometry G;

// Buffers are address ranges that are never dereferenced.  planes: two planes; third: the third plane (modes 1, 2) or
// the destination of a single step out of place (mode 3).
static float *const PLANES = reinterpret_cast<float *>(uintptr_t(1) << 40);
static float *const THIRD = reinterpret_cast<float *>(uintptr_t(2) << 40);
static std::vector<int> writes_planes, writes_third;     // stores per cell
static std::vector<char> loads_planes, loads_third;      // whether a cell was loaded
static long failures = 0, checks = 0;
static std::string current_case;

static void fail(const char *what, long a = 0, long b = 0) {
    if (++failures <= 40) std::printf("FAIL %s: %s (%ld, %ld) block %u thread %u\n", current_case.c_str(), what, a, b, blockIdx.x, threadIdx.x);
}
static void model_require(bool cond, const char *text) { if (!cond) fail(text); }

// which buffer and cell an address names; -1 when outside both
static int locate(const void *p, long &cell, long bytes) {
    const intptr_t a = reinterpret_cast<intptr_t>(p);
    const intptr_t p0 = reinterpret_cast<intptr_t>(PLANES), t0 = reinterpret_cast<intptr_t>(THIRD);
    const long plane = (long)G.ny * G.nx;
    if (a >= p0 && a + bytes <= p0 + 2 * plane * 4) { cell = (a - p0) / 4; return 0; }
    if (a >= t0 && a + bytes <= t0 + plane * 4) { cell = (a - t0) / 4; return 1; }
    return -1;
}
typedef float model_f4 __attribute__((vector_size(16)));
static void record_load(const void *p, int n) {
    long cell;
    checks++;
    const int where = locate(p, cell, 4L * n);
    if (where < 0) { fail("load outside its buffer", (long)(reinterpret_cast<intptr_t>(p) & 0xffffffffff), n); return; }
    if (n == 4 && (reinterpret_cast<intptr_t>(p) & 15)) fail("16-byte load not on a 16-byte boundary", cell);
    for (int e = 0; e < n; e++) (where == 0 ? loads_planes : loads_third)[cell + e] = 1;
}
static void record_store(const void *p, int n) {
    long cell;
    checks++;
    const int where = locate(p, cell, 4L * n);
    if (where < 0) { fail("store outside its buffer", (long)(reinterpret_cast<intptr_t>(p) & 0xffffffffff), n); return; }
    if (n == 4 && (reinterpret_cast<intptr_t>(p) & 15)) fail("16-byte store not on a 16-byte boundary", cell);
    for (int e = 0; e < n; e++) (where == 0 ? writes_planes : writes_third)[cell + e] += 1;
}
static inline model_f4 model_load4(const void *p) { record_load(p, 4); return model_f4{0.f, 0.f, 0.f, 0.f}; }
static inline float model_load1(const void *p) { record_load(p, 1); return 0.f; }

#define ST_HOST_MODEL 1
#define ST_CONSTEXPR const
#define ST_STATIC_ASSERT(cond, text) model_require((cond), text)
#define ST_SKIP_ARITHMETIC 1
#define ST_GLOBAL_LOAD4(p, stream) model_load4(p)
#define ST_GLOBAL_LOAD1(p) model_load1(p)
#define ST_GLOBAL_STORE4(p, v, stream) record_store((p), 4)
#define ST_GLOBAL_STORE1(p, v) record_store((p), 1)

#define ST_NY G.ny
#define ST_NX G.nx
#define ST_Y0 G.y0
#define ST_Y1 G.y1
#define ST_X0 G.x0
#define ST_X1 G.x1
#define ST_GX G.gx
#define ST_GY G.gy
#define ST_IBX0 G.ibx0
#define ST_IBX1 G.ibx1
#define ST_IBY0 G.iby0
#define ST_IBY1 G.iby1
#define ST_R G.r
#define ST_MODE G.mode
#define ST_W 8
#define ST_MERGE 1
#define ST_XCD 1
#define ST_OCC 0
#define ST_STREAM 2
#define ST_RAD 1
#define ST_EXPR (ST_AT(0, 0) + ST_AT(-1, 0) + ST_AT(1, 0) + ST_AT(0, -1) + ST_AT(0, 1))

// the fused form: 8 wavefronts x 11 rows, boundary slices of 5 rows per thread
#define ST_NAME model_fused
#define ST_NAME_EDGE model_fused_edge
#define ST_RPT 11
#define ST_RPT_EDGE 5
#include "../../tiramisu_amd/csrc/kernels/stencil2d_regs.hip.h"
#undef ST_NAME
#undef ST_NAME_EDGE
#undef ST_RPT
#undef ST_RPT_EDGE
// the single step out of place: 8 wavefronts x 4 rows, boundary slices of 2 rows per thread
#define ST_NAME model_single
#define ST_NAME_EDGE model_single_edge
#define ST_RPT 4
#define ST_RPT_EDGE 2
#include "../../tiramisu_amd/csrc/kernels/stencil2d_regs.hip.h"
#undef ST_NAME
#undef ST_NAME_EDGE
#undef ST_RPT
#undef ST_RPT_EDGE

// One launch of `steps` steps in `mode` reading plane `src_plane` (of the pair; mode 2 reads the third plane).
static void run_launch(int ny, int nx, int steps, int mode, int src_plane) {
    const int waves = 8, rows = mode == 3 ? 4 : 11;
    const tstencil::launch_geometry g = tstencil::plan_launch(ny, nx, 1, ny - 2, 1, nx - 2, 1, steps, waves, rows);
    if (g.rows_edge != (mode == 3 ? 2 : 5)) {
        // the emitter would compile another instance of the kernel (whole rows per thread in the slices): not modelled
        return;
    }
    G = {ny, nx, 1, ny - 2, 1, nx - 2, (int)g.tiles_x, (int)g.tiles_y, (int)g.ibx0, (int)g.ibx1, (int)g.iby0, (int)g.iby1, steps, mode};
    char text[160];
    std::snprintf(text, sizeof text, "plane %dx%d, %d step(s), mode %d, source plane %d", ny, nx, steps, mode, src_plane);
    current_case = text;
    const long plane = (long)ny * nx;
    writes_planes.assign(2 * plane, 0);
    writes_third.assign(plane, 0);
    loads_planes.assign(2 * plane, 0);
    loads_third.assign(plane, 0);
    const long grid = g.interior + g.edge_tiles * g.slices;
    for (long b = 0; b < grid; b++)
        for (unsigned t = 0; t < 64u * waves; t++) {
            blockIdx = {(unsigned)b, 0, 0};
            threadIdx = {t, 0, 0};
            if (mode == 3) model_single(PLANES, src_plane, THIRD);
            else model_fused(PLANES, src_plane, THIRD);
        }
    // ---- what the launch owes
    auto in_domain = [&](long y, long x) { return y >= 1 && y <= ny - 2 && x >= 1 && x <= nx - 2; };
    const int dst_plane = (src_plane + steps) & 1, prev_plane = (src_plane + steps - 1) & 1;
    for (long y = 0; y < ny; y++)
        for (long x = 0; x < nx; x++) {
            const long c = y * nx + x;
            const bool dom = in_domain(y, x);
            int want_plane[2] = {0, 0}, want_third = 0;
            if (mode == 0) want_plane[dst_plane] = dom;
            if (mode == 1) want_third = 1;
            if (mode == 2) { want_plane[dst_plane] += dom; want_plane[prev_plane] += dom; }
            if (mode == 3) want_third = dom;
            for (int p = 0; p < 2; p++)
                if (writes_planes[p * plane + c] != want_plane[p]) fail("cell of a plane written a wrong number of times", p * plane + c, writes_planes[p * plane + c]);
            if (writes_third[c] != want_third) fail("cell of the third plane / destination written a wrong number of times", c, writes_third[c]);
        }
    // the source must be covered: every domain cell's stencil neighbourhood was loaded from the source
    for (long y = 1; y <= ny - 2; y++)
        for (long x = 1; x <= nx - 2; x++) {
            const long c = y * nx + x;
            const bool loaded = mode == 2 ? loads_third[c] : loads_planes[src_plane * plane + c];
            if (!loaded) { fail("a cell of the iteration domain is never loaded from the source", c); y = ny; break; }
        }
}

// A whole time loop: which step each plane holds after every launch of the emitter's plan.
static void run_time_loop(long first, long steps, int wanted_cap, bool third_plane_allowed) {
    const int rcap = tstencil::step_cap(wanted_cap, 1, 8 * 11);
    const bool temp_plane = steps >= 3 && third_plane_allowed;
    const std::vector<tstencil::chunk> plan = tstencil::plan_time_loop(first, steps, rcap, false, temp_plane);
    char text[160];
    std::snprintf(text, sizeof text, "time loop of %ld step(s) from step %ld, cap %d, third plane %d", steps, first, wanted_cap, (int)temp_plane);
    current_case = text;
    auto par = [](long s) { return (int)(((s % 2) + 2) % 2); };
    long holds[2], third = -1000000;     // the step whose values a plane holds
    holds[par(first - 1)] = first - 1;
    holds[par(first)] = first - 2;
    long at = first;
    for (const tstencil::chunk &c : plan) {
        checks++;
        if (c.first != at) fail("launches do not follow one another", c.first, at);
        const int src = par(c.first - 1);
        if (c.mode == 2 ? third != c.first - 1 : holds[src] != c.first - 1) fail("a launch reads a plane that does not hold the step before its first", c.first, c.mode);
        if ((c.mode == 0 || c.mode == 1) && c.steps % 2 != 1) fail("a launch between the planes advances an even number of steps", c.steps);
        if (c.mode == 2 && c.steps < 2) fail("the final launch advances fewer than two steps", c.steps);
        if (c.steps > rcap || c.steps < 1) fail("a launch exceeds the cap", c.steps, rcap);
        const long last = c.first + c.steps - 1;
        if (c.mode == 0) holds[par(last)] = last;
        if (c.mode == 1) third = last;
        if (c.mode == 2) { holds[par(last)] = last; holds[par(last - 1)] = last - 1; }
        at = last + 1;
    }
    const long end = first + steps - 1;
    if (at != end + 1) fail("the launches do not cover the time loop", at, end);
    if (holds[par(end)] != end) fail("the last step is not in the plane of its parity", holds[par(end)], end);
    if (steps >= 2 && holds[par(end - 1)] != end - 1) fail("the last step but one is not in the other plane", holds[par(end - 1)], end - 1);
}

int main(int argc, char **argv) {
    const int n_lo = argc > 1 ? std::atoi(argv[1]) : 5, n_hi = argc > 2 ? std::atoi(argv[2]) : 300;
    const int r_hi = argc > 3 ? std::atoi(argv[3]) : 13;
    long launches = 0;
    for (int n = n_lo; n <= n_hi; n++) {
        // square planes, and some with more columns than rows so that the two extents meet different residues mod 4
        std::vector<int> widths = {n};
        if (n <= 64 || n % 7 == 0) widths.push_back(n + 3 + n % 5);
        for (int nx : widths) {
            const int ny = n;
            for (int r = 1; r <= r_hi; r++) {
                if (88 - 2 * r <= 0) break;
                for (int mode = 0; mode <= 3; mode++) {
                    if ((mode == 0 || mode == 1) && r % 2 == 0) continue;
                    if (mode == 2 && r < 2) continue;
                    if (mode == 3 && r != 1) continue;
                    for (int src = 0; src < 2; src++) {
                        if (src == 1 && n > 48) continue;          // the source plane only moves addresses by one plane
                        run_launch(ny, nx, r, mode, src);
                        launches++;
                    }
                }
            }
        }
    }
    long loops = 0;
    for (long steps = 1; steps <= 64; steps++)
        for (int cap : {1, 2, 3, 4, 5, 8, 11, 12, 13, 20})
            for (int third = 0; third < 2; third++)
                for (long first : {1L, 2L, 0L, -3L}) { run_time_loop(first, steps, cap, third != 0); loops++; }
    std::printf("%ld launches and %ld time loops modelled, %ld accesses and plan steps checked, %ld failure(s)\n", launches, loops, checks, failures);
    return failures ? 1 : 0;
}
