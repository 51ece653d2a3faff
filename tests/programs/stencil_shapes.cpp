// Stencils other than the 5-point heat kernel, to exercise the time-tiled stencil back-end:
//   box9_<NY>x<NX>x<STEPS>   radius 1 with diagonal taps (a weighted 3x3 box, as in the reference's
//                            image blurs, benchmarks/halide/blurxy_tiramisu.cpp, iterated in time),
//   far2_<NY>x<NX>x<STEPS>   radius 2: taps two cells away along both axes and two diagonal taps.
// Planes are rectangular (NY rows, NX columns) and ping-pong on t % 2; a margin of the stencil's
// radius is the fixed boundary.  Built for the GPU, or with -DTIRAMISU_TARGET_CPU for the CPU code
// the tests compare with.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

static void finish(computation &S, buffer &planes, var y, var x, const std::string &name)
{
#ifdef TIRAMISU_TARGET_CPU
    S.parallelize(y);
    tiramisu::codegen({&planes}, "build/" + name + "_cpu.o", false);
#else
    planes.tag_gpu_global();
    var yb("yb"), xb("xb"), yt("yt"), xt("xt");
    S.gpu_tile(y, x, 8, 32, yb, xb, yt, xt);
    tiramisu::codegen({&planes}, "build/" + name + ".o", true);
#endif
}

static void box9(int NY, int NX, int STEPS)
{
    const std::string name = "box9_" + std::to_string(NY) + "x" + std::to_string(NX) + "x" + std::to_string(STEPS);
    tiramisu::init(name);
    var t("t", 1, STEPS + 1), y("y", 1, NY - 1), x("x", 1, NX - 1);
    buffer planes("planes", {2, NY, NX}, p_float32, a_output);
    computation S("S", {t, y, x}, p_float32);
    S.set_expression(S(t - 1, y, x) * 0.25f +
                     (S(t - 1, y - 1, x) + S(t - 1, y + 1, x) + S(t - 1, y, x - 1) + S(t - 1, y, x + 1)) * 0.125f +
                     (S(t - 1, y - 1, x - 1) + S(t - 1, y - 1, x + 1) + S(t - 1, y + 1, x - 1) + S(t - 1, y + 1, x + 1)) * 0.0625f);
    S.store_in(&planes, {t % 2, y, x});
    finish(S, planes, y, x, name);
}

static void far2(int NY, int NX, int STEPS)
{
    const std::string name = "far2_" + std::to_string(NY) + "x" + std::to_string(NX) + "x" + std::to_string(STEPS);
    tiramisu::init(name);
    var t("t", 1, STEPS + 1), y("y", 2, NY - 2), x("x", 2, NX - 2);
    buffer planes("planes", {2, NY, NX}, p_float32, a_output);
    computation S("S", {t, y, x}, p_float32);
    S.set_expression(S(t - 1, y, x) * 0.5f +
                     (S(t - 1, y - 2, x) + S(t - 1, y + 2, x) + S(t - 1, y, x - 2) + S(t - 1, y, x + 2)) * 0.0625f +
                     (S(t - 1, y - 1, x + 1) + S(t - 1, y + 1, x - 1)) * 0.125f);
    S.store_in(&planes, {t % 2, y, x});
    finish(S, planes, y, x, name);
}

int main()
{
    box9(200, 520, 6);    // several tiles in both directions, interior workgroups
    box9(45, 39, 3);      // rows not a multiple of 4 elements
    far2(200, 520, 5);
    far2(70, 50, 4);
    return 0;
}
