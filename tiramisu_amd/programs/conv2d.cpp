// conv2d + bias + ReLU, NCHW fp32, 3x3 kernel, stride 1, padding 1:
//   out[n, co, y, x] = max(0, bias[co] + sum_{ci,ky,kx} in_pad[n, ci, y+ky, x+kx] * w[co, ci, ky, kx])
// The padding is materialised by the caller: the input argument is the (H+2) x (W+2) padded
// tensor, as in the reference's direct convolution
// (benchmarks/DNN/layers/convolution/direct/cpu/conv_layer_generator_tiramisu.cpp:19-21); the
// loop nest is the NCHW form of benchmarks/auto-scheduler_benchmarks/convolution/
// convolution_generator.cpp:17-25 and ReLU is expr(o_max, x, 0) as in
// benchmarks/DNN/layers/relu/cpu/relu_layer_generator_tiramisu.cpp:20.
//
// GPU schedule: (y, x) tiled 16x16 onto threads, (n, co, y-tile) onto blocks, the x-tile loop
// and the reduction serial in the thread, a register accumulator, initialisation (bias),
// reduction and ReLU fused in the thread.  The HIP back-end proves the nest to be a dense
// contraction with M = {co}, N = {n, y, x}, K = {ci, ky, kx} and emits an implicit-GEMM MFMA
// kernel whose B operand gathers the im2col view of the padded input into LDS.
// CPU schedule (-DTIRAMISU_TARGET_CPU): parallelize n and co, vectorize x by 8 (the tags of
// conv_layer_generator_tiramisu.cpp:110-112,172-173).
// One generated function per shape: conv2d_<N>x<Cin>x<Cout>x<H>.
#include <cstdlib>
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

static void generate(int NB, int CI, int CO, int H)
{
    const int W = H;
    const std::string name = "conv2d_" + std::to_string(NB) + "x" + std::to_string(CI) + "x" + std::to_string(CO) + "x" + std::to_string(H);
    tiramisu::init(name);

    var n("n", 0, NB), co("co", 0, CO), y("y", 0, H), x("x", 0, W), ci("ci", 0, CI), ky("ky", 0, 3), kx("kx", 0, 3);
    var yp("yp", 0, H + 2), xp("xp", 0, W + 2);

    buffer b_in("b_in", {NB, CI, H + 2, W + 2}, p_float32, a_input);
    buffer b_w("b_w", {CO, CI, 3, 3}, p_float32, a_input);
    buffer b_bias("b_bias", {CO}, p_float32, a_input);
    buffer b_out("b_out", {NB, CO, H, W}, p_float32, a_output);

    input in("in", {n, ci, yp, xp}, p_float32);
    input w("w", {co, ci, ky, kx}, p_float32);
    input bias("bias", {co}, p_float32);
    in.store_in(&b_in);
    w.store_in(&b_w);
    bias.store_in(&b_bias);

    computation conv_init("conv_init", {n, co, y, x}, bias(co));
    computation conv("conv", {n, co, y, x, ci, ky, kx}, p_float32);
    conv.set_expression(conv(n, co, y, x, 0, 0, 0) + in(n, ci, y + ky, x + kx) * w(co, ci, ky, kx));
    computation relu("relu", {n, co, y, x}, expr(o_max, conv(n, co, y, x, 0, 0, 0), expr((float)0)));
    relu.store_in(&b_out);

#ifdef TIRAMISU_TARGET_CPU
    conv_init.store_in(&b_out);
    conv.store_in(&b_out, {n, co, y, x});
    conv_init.parallelize(n);
    conv.parallelize(n);
    relu.parallelize(n);
    // x innermost for the vector loop: (n, co, y, ci, ky, kx, x)
    conv.interchange(x, ci);
    conv.interchange(x, ky);
    conv.interchange(x, kx);
    var xo("xo"), xi("xi");
    if (W % 8 == 0) conv.vectorize(x, 8, xo, xi);
    conv_init.then(conv, computation::root).then(relu, computation::root);
    tiramisu::codegen({&b_in, &b_w, &b_bias, &b_out}, "build/" + name + "_cpu.o", false);
#else
    b_in.tag_gpu_global();
    b_w.tag_gpu_global();
    b_bias.tag_gpu_global();
    b_out.tag_gpu_global();
    buffer acc_reg("acc_reg", {1}, p_float32, a_temporary);
    acc_reg.tag_gpu_register();
    computation acc_decl("acc_decl", {n, co, y, x}, allocate(acc_reg));
    conv_init.store_in(&acc_reg, {0});
    conv.store_in(&acc_reg, {0});
    var yb("yb"), xb("xb"), yt("yt"), xt("xt");
    const int T = (H % 16 == 0) ? 16 : 4;
    for (computation *c : {&acc_decl, &conv_init, &conv, &relu}) {
        c->tile(y, x, T, T, yb, xb, yt, xt);
        // loop levels are now n, co, yb, xb, yt, xt: blocks (n, co, yb), threads (yt, xt); the xb
        // loop stays serial inside the kernel
        c->tag_gpu_block_level(0, 1, 2);
        c->tag_gpu_thread_level(4, 5);
    }
    acc_decl.then(conv_init, xt).then(conv, xt).then(relu, xt);
    tiramisu::codegen({&b_in, &b_w, &b_bias, &b_out}, "build/" + name + ".o", true);
#endif
}

int main(int argc, char **argv)
{
    tiramisu::backend_options_from_command_line(argc, argv);
    if (const char *nb = std::getenv("CONV_ONLY_FULL")) {   // experiments: the benchmark shape alone, with another batch size
        generate(std::atoi(nb) > 1 ? std::atoi(nb) : 32, 64, 64, 112);
        return 0;
    }
    generate(32, 64, 64, 112);   // benchmark configuration 4
    generate(2, 8, 64, 16);
    generate(1, 3, 5, 12);       // ragged in every group
    generate(3, 4, 32, 8);
    return 0;
}
