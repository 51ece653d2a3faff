// Bilinear resampling of an image along an affine map, with the sample position, its integer
// cell and the interpolation weights as constants computed inside the loop nest (scalars declared
// at a loop level, not function-wide) and data-dependent, clamped indices into the input.
// Features of the reference's benchmarks/halide/warp_affinegpu_tiramisu.cpp:55-76 (constants
// with function_wide = false, clamp, floor, casts, non-affine accesses), on a program of its own.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

int main()
{
    const int H = 90, W = 132;
    tiramisu::init("resample_bilinear");
    function *fct = global::get_implicit_function();

    var y("y", 0, H), x("x", 0, W);
    var yb("yb"), xb("xb"), yt("yt"), xt("xt");
    buffer src("src", {H, W}, p_uint8, a_input);
    buffer dst("dst", {H, W}, p_float32, a_output);
    src.tag_gpu_global();
    dst.tag_gpu_global();
    input pix("pix", {y, x}, p_uint8);
    pix.store_in(&src);

    computation out("out", {y, x}, p_float32);
    // sample position (a slight rotation and shift), per output pixel: level 1 = the x loop
    constant fy("fy", cast(p_float32, y) * 0.96875f + cast(p_float32, x) * 0.0625f - 1.5f, p_float32, false, &out, 1, fct);
    constant fx("fx", cast(p_float32, x) * 0.96875f - cast(p_float32, y) * 0.0625f + 2.25f, p_float32, false, &out, 1, fct);
    constant y0("y0", cast(p_int32, floor(fy)), p_int32, false, &out, 1, fct);
    constant x0("x0", cast(p_int32, floor(fx)), p_int32, false, &out, 1, fct);
    constant wy("wy", expr(fy) - floor(fy), p_float32, false, &out, 1, fct);
    constant wx("wx", expr(fx) - floor(fx), p_float32, false, &out, 1, fct);
    constant ya("ya", clamp(y0, 0, H - 1), p_int32, false, &out, 1, fct);
    constant yc("yc", clamp(y0 + 1, 0, H - 1), p_int32, false, &out, 1, fct);
    constant xa("xa", clamp(x0, 0, W - 1), p_int32, false, &out, 1, fct);
    constant xc("xc", clamp(x0 + 1, 0, W - 1), p_int32, false, &out, 1, fct);

    expr p00 = cast(p_float32, pix(ya, xa)), p01 = cast(p_float32, pix(ya, xc));
    expr p10 = cast(p_float32, pix(yc, xa)), p11 = cast(p_float32, pix(yc, xc));
    expr top = p00 + (p01 - p00) * wx, bottom = p10 + (p11 - p10) * wx;
    out.set_expression(top + (bottom - top) * wy);
    out.store_in(&dst);

    // every constant lives in the same (tiled, GPU-mapped) loop nest as its consumer
    block({&fy, &fx, &y0, &x0, &wy, &wx, &ya, &yc, &xa, &xc, &out}).gpu_tile(y, x, 8, 32, yb, xb, yt, xt);
    fy.then(fx, xt).then(y0, xt).then(x0, xt).then(wy, xt).then(wx, xt).then(ya, xt).then(yc, xt).then(xa, xt).then(xc, xt).then(out, xt);

    tiramisu::codegen({&src, &dst}, "build/resample_bilinear.o", true);
    return 0;
}
