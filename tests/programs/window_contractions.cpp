// Contractions whose gathered operand is a window sliding over a tensor, in shapes other than the benchmark's 3x3
// convolution: a 1-D convolution with 9 taps, a 5x5 convolution over rectangular images, a 3x3 convolution whose
// tiles do not fill a round of the launch's workgroups (so the last tiles are cut into pieces), and a 3x3
// convolution whose channel count admits only blocks of 4 channels.  out = bias + sum over (channel, taps), no
// clamp, so that every sum shows in the result.  One function each: window_<name>.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

// out[n, co, x] = bias[co] + sum_{ci, k} in[n, ci, x + k] * w[co, ci, k]
static void conv1d(const std::string &name, int NB, int CI, int CO, int X, int TAPS)
{
    tiramisu::init(name);
    var n("n", 0, NB), co("co", 0, CO), x("x", 0, X), ci("ci", 0, CI), k("k", 0, TAPS), xp("xp", 0, X + TAPS - 1);
    buffer b_in("b_in", {NB, CI, X + TAPS - 1}, p_float32, a_input), b_w("b_w", {CO, CI, TAPS}, p_float32, a_input);
    buffer b_bias("b_bias", {CO}, p_float32, a_input), b_out("b_out", {NB, CO, X}, p_float32, a_output);
    input in("in", {n, ci, xp}, p_float32), w("w", {co, ci, k}, p_float32), bias("bias", {co}, p_float32);
    in.store_in(&b_in);
    w.store_in(&b_w);
    bias.store_in(&b_bias);
    computation init_("init_", {n, co, x}, bias(co));
    computation conv("conv", {n, co, x, ci, k}, p_float32);
    conv.set_expression(conv(n, co, x, 0, 0) + in(n, ci, x + k) * w(co, ci, k));
    init_.store_in(&b_out);
    conv.store_in(&b_out, {n, co, x});
#ifdef TIRAMISU_TARGET_CPU
    init_.then(conv, computation::root);
    tiramisu::codegen({&b_in, &b_w, &b_bias, &b_out}, "build/" + name + "_cpu.o", false);
#else
    for (buffer *b : {&b_in, &b_w, &b_bias, &b_out}) b->tag_gpu_global();
    var xb("xb"), xt("xt");
    for (computation *c : {&init_, &conv}) {
        c->split(x, 64, xb, xt);
        c->tag_gpu_block_level(0, 1, 2);
        c->tag_gpu_thread_level(3);
    }
    init_.then(conv, xt);
    tiramisu::codegen({&b_in, &b_w, &b_bias, &b_out}, "build/" + name + ".o", true);
#endif
}

// out[n, co, y, x] = bias[co] + sum_{ci, ky, kx} in[n, ci, y + ky, x + kx] * w[co, ci, ky, kx], images of H x W
static void conv2d(const std::string &name, int NB, int CI, int CO, int H, int W, int KH, int KW)
{
    tiramisu::init(name);
    var n("n", 0, NB), co("co", 0, CO), y("y", 0, H), x("x", 0, W), ci("ci", 0, CI), ky("ky", 0, KH), kx("kx", 0, KW);
    var yp("yp", 0, H + KH - 1), xp("xp", 0, W + KW - 1);
    buffer b_in("b_in", {NB, CI, H + KH - 1, W + KW - 1}, p_float32, a_input), b_w("b_w", {CO, CI, KH, KW}, p_float32, a_input);
    buffer b_bias("b_bias", {CO}, p_float32, a_input), b_out("b_out", {NB, CO, H, W}, p_float32, a_output);
    input in("in", {n, ci, yp, xp}, p_float32), w("w", {co, ci, ky, kx}, p_float32), bias("bias", {co}, p_float32);
    in.store_in(&b_in);
    w.store_in(&b_w);
    bias.store_in(&b_bias);
    computation init_("init_", {n, co, y, x}, bias(co));
    computation conv("conv", {n, co, y, x, ci, ky, kx}, p_float32);
    conv.set_expression(conv(n, co, y, x, 0, 0, 0) + in(n, ci, y + ky, x + kx) * w(co, ci, ky, kx));
    init_.store_in(&b_out);
    conv.store_in(&b_out, {n, co, y, x});
#ifdef TIRAMISU_TARGET_CPU
    init_.then(conv, computation::root);
    tiramisu::codegen({&b_in, &b_w, &b_bias, &b_out}, "build/" + name + "_cpu.o", false);
#else
    for (buffer *b : {&b_in, &b_w, &b_bias, &b_out}) b->tag_gpu_global();
    var yb("yb"), xb("xb"), yt("yt"), xt("xt");
    for (computation *c : {&init_, &conv}) {
        c->tile(y, x, 8, 8, yb, xb, yt, xt);
        c->tag_gpu_block_level(0, 1, 2);        // n, co, yb; the xb loop stays serial in the thread
        c->tag_gpu_thread_level(4, 5);
    }
    init_.then(conv, xt);
    tiramisu::codegen({&b_in, &b_w, &b_bias, &b_out}, "build/" + name + ".o", true);
#endif
}

int main()
{
    conv1d("window_conv1d_9", 6, 16, 64, 1024, 9);             // rows of 1032 floats, two blocks of 8 channels
    conv2d("window_conv2d_5x5", 3, 8, 128, 24, 32, 5, 5);       // rectangular 24 x 32 images, two tile rows (M = 128)
    conv2d("window_conv2d_3x3_pieces", 129, 16, 64, 32, 32, 3, 3);   // 516 tiles of 64 x 256 on 512 workgroups: 4 tiles cut into pieces
    conv2d("window_conv2d_3x3_c4", 2, 4, 64, 16, 16, 3, 3);     // 4 channels: one block of 4
    return 0;
}
