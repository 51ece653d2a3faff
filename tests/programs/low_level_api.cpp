// NO_CPU_VARIANT (the hand-driven pipeline names its back-end itself; the expected result is a closed form)
// The low-level interface: an explicit tiramisu::function, a function-wide constant built with
// the long constructor, a computation given by an isl iteration-domain string and an isl access
// relation, a three-dimensional gpu_tile, and the hand-driven pipeline (set_arguments,
// gen_time_space_domain, gen_isl_ast, gen_cuda_stmt, gen_halide_stmt, gen_halide_obj) instead of
// codegen().  Same calls as the reference's tests/test_19.cpp:19-45 (gpu_tile with three loops)
// and benchmarks/halide/gaussiangpu_tiramisu.cpp:96-103 (pipeline), on a program of its own:
// S(i, j, k) = i + 2*j + 3*k summed over k into out[i][j] ... kept simple: out[i][k] = 7 for the
// last j, written by every j (the same value), as test_19 does with its middle loop.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

int main()
{
    const int SIZE = 10;
    tiramisu::global::set_default_tiramisu_options();
    tiramisu::function fill3d("low_level_api");
    tiramisu::constant N("N", tiramisu::expr((int32_t)SIZE), p_int32, true, NULL, 0, &fill3d);
    tiramisu::var i0("i0"), i1("i1"), i2("i2");
    tiramisu::buffer grid("grid", {SIZE, SIZE}, tiramisu::p_int32, a_output, &fill3d);
    grid.tag_gpu_global();
    // the value depends on the two stored indices only, so every i1 writes the same thing
    tiramisu::computation S0("[N]->{S0[i0,i1,i2]: 0<=i0<N and 0<=i1<N and 0<=i2<N}",
                             tiramisu::expr(i0) * 100 + tiramisu::expr(i2) + 7, true, p_int32, &fill3d);
    S0.set_access("[N]->{S0[i0,i1,i2]->grid[i0,i2]}");
    S0.gpu_tile(i0, i1, i2, 2, 2, 4);   // 10 is not a multiple of 4: guarded last tile

    fill3d.set_arguments({&grid});
    fill3d.gen_time_space_domain();
    fill3d.gen_isl_ast();
    fill3d.gen_cuda_stmt();
    fill3d.gen_halide_stmt();
    fill3d.gen_halide_obj("build/low_level_api.o");
    return 0;
}
