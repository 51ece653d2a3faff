// out(y, x) = in(y, x) on an 8192 x 8192 fp32 plane, both buffers GPU-resident: a plain copy of known
// size (256 MiB read, 256 MiB written).  The benchmark uses it to calibrate hardware byte counters and to
// compare what the two emitters make of a streaming kernel with the vendor's device-to-device copy:
//   copy_plane        the schedule-faithful emitter: one element per thread, as the schedule says
//                     (the single-step stencil form is switched off through a back-end option);
//   copy_plane_quads  the same program left to the back-end: a point-wise map of one buffer into another is
//                     a stencil of radius 0 taken by the stencil emitter's single-step form -- 16 bytes per
//                     lane, four rows per thread, stores with the non-temporal hint.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

static void generate(const std::string &name, bool as_scheduled)
{
    const int N = 8192;
    tiramisu::init(name);
    if (as_scheduled) tiramisu::set_backend_option("no_single_step_stencil", "1");
    var y("y", 0, N), x("x", 0, N);
    buffer src("src", {N, N}, p_float32, a_input);
    buffer dst("dst", {N, N}, p_float32, a_output);
    src.tag_gpu_global();
    dst.tag_gpu_global();
    input in("in", {y, x}, p_float32);
    in.store_in(&src);
    computation out("out", {y, x}, in(y, x));
    out.store_in(&dst);
    var yb("yb"), xb("xb"), yt("yt"), xt("xt");
    out.gpu_tile(y, x, 4, 64, yb, xb, yt, xt);
    tiramisu::codegen({&src, &dst}, "build/" + name + ".o", true);
}

int main()
{
    generate("copy_plane", true);
    generate("copy_plane_quads", false);
    return 0;
}
