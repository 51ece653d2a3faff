// copy_plane: out(y, x) = in(y, x) on an 8192 x 8192 fp32 plane, both buffers GPU-resident.
// A plain copy of known size (256 MiB read, 256 MiB written) compiled by the schedule-faithful
// emitter; the benchmark uses it to calibrate hardware byte counters and as a measured
// ceiling for streaming kernels on this device.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

int main()
{
    const int N = 8192;
    tiramisu::init("copy_plane");
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
    tiramisu::codegen({&src, &dst}, "build/copy_plane.o", true);
    return 0;
}
