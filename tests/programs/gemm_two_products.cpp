// out(b, i, j) = bias(j) + sum over k of (W(j, k) * x(b, i, k) + R(j, k) * h(b, i, k)): a contraction whose
// update adds two products per reduction step (the merged form of a recurrent cell's gates,
// benchmarks/DNN/blocks/LSTM/gpu/generator.cpp:110-118 computes the two halves one after the
// other), with a batch dimension mapped to a third block index and the bias as fused
// initialisation.  One function: gemm_two_products.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

int main()
{
    const int NB = 3, M = 64, N = 96, K = 80;
    tiramisu::init("gemm_two_products");

    var b("b", 0, NB), i("i", 0, M), j("j", 0, N), k("k", 0, K);
    var ib("ib"), it("it"), jb("jb"), jt("jt");

    buffer buf_W("buf_W", {N, K}, p_float32, a_input), buf_R("buf_R", {N, K}, p_float32, a_input);
    buffer buf_x("buf_x", {NB, M, K}, p_float32, a_input), buf_h("buf_h", {NB, M, K}, p_float32, a_input);
    buffer buf_bias("buf_bias", {N}, p_float32, a_input);
    buffer buf_out("buf_out", {NB, M, N}, p_float32, a_output);
    for (buffer *q : {&buf_W, &buf_R, &buf_x, &buf_h, &buf_bias, &buf_out}) q->tag_gpu_global();

    input W("W", {j, k}, p_float32), R("R", {j, k}, p_float32);
    input x("x", {b, i, k}, p_float32), h("h", {b, i, k}, p_float32);
    input bias("bias", {j}, p_float32);
    W.store_in(&buf_W);
    R.store_in(&buf_R);
    x.store_in(&buf_x);
    h.store_in(&buf_h);
    bias.store_in(&buf_bias);

    computation out_init("out_init", {b, i, j}, bias(j));
    computation out("out", {b, i, j, k}, p_float32);
    out.set_expression(out(b, i, j, 0) + W(j, k) * x(b, i, k) + R(j, k) * h(b, i, k));
    out_init.store_in(&buf_out, {b, i, j});
    out.store_in(&buf_out, {b, i, j});

    for (computation *c : {&out_init, &out}) {
        c->tile(i, j, 16, 16, ib, jb, it, jt);
        c->tag_gpu_block_level(0, 1, 2);
        c->tag_gpu_thread_level(3, 4);
    }
    out_init.then(out, jt);

    tiramisu::codegen({&buf_W, &buf_R, &buf_x, &buf_h, &buf_bias, &buf_out}, "build/gemm_two_products.o", true);
    return 0;
}
