// One 5-point sweep out of place on the benchmark's plane size: out(y, x) = 0.3 in(y, x) + 0.4 (n + s + w + e) on the
// interior of 8192 x 8192 floats, the weights of the reference's heat2d (benchmarks/halide/heat2d_tiramisu.cpp:52-86),
// input and output in buffers of their own.  Taken by the stencil back-end as a single step out of place; it is
// `bench.py --workload sweep5` (not part of the default run) and the smaller shapes of
// tests/programs/stencil_single_step.cpp are its parity cases.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

int main(int argc, char **argv)
{
    tiramisu::backend_options_from_command_line(argc, argv);
    const int N = 8192;
    tiramisu::init("sweep5_8192x8192");
    var yy("yy", 0, N), xx("xx", 0, N), y("y", 1, N - 1), x("x", 1, N - 1);
    buffer b_in("b_in", {N, N}, p_float32, a_input), b_out("b_out", {N, N}, p_float32, a_output);
    input in("in", {yy, xx}, p_float32);
    in.store_in(&b_in, {yy, xx});
    computation S("S", {y, x}, in(y, x) * 0.3f + (in(y - 1, x) + in(y + 1, x) + in(y, x - 1) + in(y, x + 1)) * 0.4f);
    S.store_in(&b_out, {y, x});
#ifdef TIRAMISU_TARGET_CPU
    S.parallelize(y);
    tiramisu::codegen({&b_in, &b_out}, "build/sweep5_8192x8192_cpu.o", false);
#else
    b_in.tag_gpu_global();
    b_out.tag_gpu_global();
    var yb("yb"), xb("xb"), yt("yt"), xt("xt");
    S.gpu_tile(y, x, 16, 16, yb, xb, yt, xt);
    tiramisu::codegen({&b_in, &b_out}, "build/sweep5_8192x8192.o", true);
#endif
    return 0;
}
