// One stencil step out of place: out(y, x) = f(in(y + dy, x + dx)) on the interior of a plane, input and output in
// buffers of their own -- the shape of the reference's single-sweep programs (benchmarks/halide/heat2d_tiramisu.cpp,
// the 3 x 3 blurs) when they are written without hand-staged LDS tiles.  The stencil back-end takes the nest
// (one read of the plane through registers and lane shifts, one write) instead of one thread per point.
//   sweep5_<NY>x<NX>   0.3 c + 0.4 (n + s + w + e), margin 1 (the weights of the reference's heat2d)
//   wide9_<NY>x<NX>    radius 2 with two diagonal taps, margin 2
// Cells of the output outside the iteration domain are not written.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

static void finish(computation &S, buffer &b_in, buffer &b_out, var y, var x, const std::string &name)
{
#ifdef TIRAMISU_TARGET_CPU
    S.parallelize(y);
    tiramisu::codegen({&b_in, &b_out}, "build/" + name + "_cpu.o", false);
#else
    b_in.tag_gpu_global();
    b_out.tag_gpu_global();
    var yb("yb"), xb("xb"), yt("yt"), xt("xt");
    S.gpu_tile(y, x, 16, 16, yb, xb, yt, xt);
    tiramisu::codegen({&b_in, &b_out}, "build/" + name + ".o", true);
#endif
}

static void sweep5(int NY, int NX)
{
    const std::string name = "sweep5_" + std::to_string(NY) + "x" + std::to_string(NX);
    tiramisu::init(name);
    var yy("yy", 0, NY), xx("xx", 0, NX), y("y", 1, NY - 1), x("x", 1, NX - 1);
    buffer b_in("b_in", {NY, NX}, p_float32, a_input), b_out("b_out", {NY, NX}, p_float32, a_output);
    input in("in", {yy, xx}, p_float32);
    in.store_in(&b_in, {yy, xx});
    computation S("S", {y, x}, in(y, x) * 0.3f + (in(y - 1, x) + in(y + 1, x) + in(y, x - 1) + in(y, x + 1)) * 0.4f);
    S.store_in(&b_out, {y, x});
    finish(S, b_in, b_out, y, x, name);
}

static void wide9(int NY, int NX)
{
    const std::string name = "wide9_" + std::to_string(NY) + "x" + std::to_string(NX);
    tiramisu::init(name);
    var yy("yy", 0, NY), xx("xx", 0, NX), y("y", 2, NY - 2), x("x", 2, NX - 2);
    buffer b_in("b_in", {NY, NX}, p_float32, a_input), b_out("b_out", {NY, NX}, p_float32, a_output);
    input in("in", {yy, xx}, p_float32);
    in.store_in(&b_in, {yy, xx});
    computation S("S", {y, x}, in(y, x) * 0.5f + (in(y - 2, x) + in(y + 2, x) + in(y, x - 2) + in(y, x + 2)) * 0.0625f +
                                   (in(y - 1, x + 1) + in(y + 1, x - 1)) * 0.125f);
    S.store_in(&b_out, {y, x});
    finish(S, b_in, b_out, y, x, name);
}

int main()
{
    sweep5(300, 520);
    sweep5(45, 39);       // rows not a multiple of 4 elements: element loads
    wide9(200, 520);
    wide9(70, 50);
    return 0;
}
