// heat2d: 5-point stencil out = 0.2 * (c + n + s + w + e) on an N x N grid with a fixed
// boundary, STEPS time steps on a ping-pong pair of planes (plane t % 2 holds step t; step 0 is
// the caller's initial grid in plane 0).  Written in the time-loop style of the reference's
// benchmarks/halide/heat3d_tiramisu.cpp:27-45; the single-step variants are
// benchmarks/halide/heat2d_tiramisu.cpp:52-86 (CPU schedule :83-86) and heat2dgpu_tiramisu.cpp.
//
// GPU schedule: time on the host, (y, x) tiled 16x16 onto blocks and threads; the buffer is a
// GPU-resident argument.  CPU schedule (built with -DTIRAMISU_TARGET_CPU): parallelize y,
// vectorize x by 8.  One generated function per (N, STEPS) instance: heat2d_<N>x<STEPS>.
#include <tiramisu/tiramisu.h>

#include <cstdlib>

using namespace tiramisu;

static void generate(int N, int STEPS)
{
    const std::string name = "heat2d_" + std::to_string(N) + "x" + std::to_string(STEPS);
    tiramisu::init(name);

    var t("t", 1, STEPS + 1), y("y", 1, N - 1), x("x", 1, N - 1);
    buffer planes("planes", {2, N, N}, p_float32, a_output);

    computation heat("heat", {t, y, x}, p_float32);
    heat.set_expression((heat(t - 1, y, x) + heat(t - 1, y - 1, x) + heat(t - 1, y + 1, x) +
                         heat(t - 1, y, x - 1) + heat(t - 1, y, x + 1)) * 0.2f);
    heat.store_in(&planes, {t % 2, y, x});

#ifdef TIRAMISU_TARGET_CPU
    var xo("xo"), xi("xi");
    heat.parallelize(y);
    if ((N - 2) % 8 == 0 || N > 64) heat.vectorize(x, 8, xo, xi);
    tiramisu::codegen({&planes}, "build/" + name + "_cpu.o", false);
#else
    planes.tag_gpu_global();
    var yb("yb"), xb("xb"), yt("yt"), xt("xt");
    heat.gpu_tile(y, x, 16, 16, yb, xb, yt, xt);
    tiramisu::codegen({&planes}, "build/" + name + ".o", true);
#endif
}

int main(int argc, char **argv)
{
    tiramisu::backend_options_from_command_line(argc, argv);
    generate(8192, 32);   // the benchmark configuration
    if (std::getenv("HEAT2D_ONLY_FULL")) return 0;   // for sweeps over the emitter's knobs
    generate(1024, 8);
    generate(1030, 9);    // rows not a multiple of 4 elements with interior tiles: unaligned strips
    generate(256, 1);
    generate(130, 4);
    generate(66, 7);
    generate(37, 6);      // rows not a multiple of 4 elements: scalar edge path
    generate(20, 2);
    return 0;
}
