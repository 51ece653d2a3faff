// Stacked LSTM forward pass, fp32: L layers, batch B, hidden = input = H, sequence length S.
//   gates(m, l) = bias(l) + W(l) * h(m, l-1) + R(l) * h(m-1, l)        (4H values per sample)
//   i, f = sigmoid(gates[0:H]), sigmoid(gates[H:2H]);  z = tanh(gates[2H:3H]);  o = sigmoid(gates[3H:4H])
//   c(m, l) = i * z + f * c(m-1, l);   h(m, l) = tanh(c(m, l)) * o;   y(m) = h(m, L-1)
// with h(-1, l) = c(-1, l) = 0 and h(m, -1) = x(m).  Packing follows the reference's library
// variant: gate order i, f, z, o (benchmarks/DNN/blocks/LSTM/gpu_lib/generator.cpp:84-87), weight
// slot 0 = input weights W, slot 1 = recurrent weights R (:69-70, :78-79); the computation
// structure (merged 4H gate rows, h/c buffers indexed [m+1][l+1]) is that of
// benchmarks/DNN/blocks/LSTM/cpu/generator.cpp:31-60, and sigmoid is 1 / (1 + exp(-x)) (:43).
//
// GPU schedule: one cell (layer l, time step m) is two loop nests -- the gates of the cell as one
// contraction with two product terms (input weights against the layer below, recurrent weights
// against the previous step; the bias initialisation fused in), then the nine element-wise
// computations over (sample, hidden unit) -- and the back-end fuses the two into one MFMA kernel
// whose workgroups hold the four gate columns of their hidden units.  Layers and time steps are host
// loops, skewed and interchanged so that the outer loop walks the diagonals l + m and the inner one,
// tagged parallel, the independent cells of a diagonal (the traversal of the reference's library
// variant, gpu_lib/generator.cpp:120-135, at the granularity of single time steps): the back-end
// runs the cells of a diagonal as one launch.  All tensors are GPU-resident.
// CPU schedule (-DTIRAMISU_TARGET_CPU): the same computations in the reference's unscheduled order
// (cpu/generator.cpp:59-75) with the batch loop parallelized.
// One generated function per shape: lstm_<L>x<B>x<H>x<S>.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

static expr sigmoid(expr v) { return expr((float)1) / (1 + expr(o_expo, -v)); }

static void generate(int L, int B, int H, int S)
{
    const std::string name = "lstm_" + std::to_string(L) + "x" + std::to_string(B) + "x" + std::to_string(H) + "x" + std::to_string(S);
    tiramisu::init(name);

    var l("l", 0, L), m("m", 0, S), k("k", 0, B), i("i", 0, H), j("j", 0, H), g("g", 0, 4 * H);

    buffer buf_weights("buf_weights", {L, 2, 4 * H, H}, p_float32, a_input);
    buffer buf_biases("buf_biases", {L, 4 * H}, p_float32, a_input);
    buffer buf_x("buf_x", {S, B, H}, p_float32, a_input);
    buffer buf_y("buf_y", {S, B, H}, p_float32, a_output);
    buffer buf_gates("buf_gates", {L, B, 4 * H}, p_float32, a_temporary);
    buffer buf_i("buf_i", {L, B, H}, p_float32, a_temporary);
    buffer buf_f("buf_f", {L, B, H}, p_float32, a_temporary);
    buffer buf_z("buf_z", {L, B, H}, p_float32, a_temporary);
    buffer buf_o("buf_o", {L, B, H}, p_float32, a_temporary);
    buffer buf_h("buf_h", {L + 1, S + 1, B, H}, p_float32, a_temporary);
    buffer buf_c("buf_c", {L, S + 1, B, H}, p_float32, a_temporary);

    input W("W", {l, g, j}, p_float32);
    input R("R", {l, g, j}, p_float32);
    input bias("bias", {l, g}, p_float32);
    input x("x", {m, k, i}, p_float32);

    computation h("h", {l, m, k, i}, p_float32);
    computation c("c", {l, m, k, i}, p_float32);
    computation h_init("h_init", {l, k, i}, expr((float)0));
    computation c_init("c_init", {l, k, i}, expr((float)0));
    computation h_copy_x("h_copy_x", {m, k, i}, x(m, k, i));
    computation gates_init("gates_init", {l, m, k, g}, bias(l, g));
    computation gates("gates", {l, m, k, g, j}, p_float32);
    gates.set_expression(gates(l, m, k, g, 0) + W(l, g, j) * h(l - 1, m, k, j) + R(l, g, j) * h(l, m - 1, k, j));
    computation sig_i("sig_i", {l, m, k, i}, sigmoid(gates(l, m, k, i, 0)));
    computation sig_f("sig_f", {l, m, k, i}, sigmoid(gates(l, m, k, i + H, 0)));
    computation tnh_z("tnh_z", {l, m, k, i}, expr(o_tanh, gates(l, m, k, i + 2 * H, 0)));
    computation sig_o("sig_o", {l, m, k, i}, sigmoid(gates(l, m, k, i + 3 * H, 0)));
    computation mul_iz("mul_iz", {l, m, k, i}, sig_i(l, m, k, i) * tnh_z(l, m, k, i));
    computation mul_fc("mul_fc", {l, m, k, i}, sig_f(l, m, k, i) * c(l, m - 1, k, i));
    c.set_expression(mul_iz(l, m, k, i) + mul_fc(l, m, k, i));
    computation tnh_c("tnh_c", {l, m, k, i}, expr(o_tanh, c(l, m, k, i)));
    h.set_expression(tnh_c(l, m, k, i) * sig_o(l, m, k, i));
    computation y("y", {m, k, i}, h(L - 1, m, k, i));

    W.store_in(&buf_weights, {l, 0, g, j});
    R.store_in(&buf_weights, {l, 1, g, j});
    bias.store_in(&buf_biases, {l, g});
    x.store_in(&buf_x);
    y.store_in(&buf_y);
    gates_init.store_in(&buf_gates, {l, k, g});
    gates.store_in(&buf_gates, {l, k, g});
    sig_i.store_in(&buf_i, {l, k, i});
    sig_f.store_in(&buf_f, {l, k, i});
    tnh_z.store_in(&buf_z, {l, k, i});
    sig_o.store_in(&buf_o, {l, k, i});
    mul_iz.store_in(&buf_i, {l, k, i});
    mul_fc.store_in(&buf_f, {l, k, i});
    tnh_c.store_in(&buf_i, {l, k, i});
    h.store_in(&buf_h, {l + 1, m + 1, k, i});
    c.store_in(&buf_c, {l, m + 1, k, i});
    h_init.store_in(&buf_h, {l + 1, 0, k, i});
    c_init.store_in(&buf_c, {l, 0, k, i});
    h_copy_x.store_in(&buf_h, {0, m + 1, k, i});

#ifdef TIRAMISU_TARGET_CPU
    for (computation *q : {&gates_init, &gates, &sig_i, &sig_f, &tnh_z, &sig_o, &mul_iz, &mul_fc, &c, &tnh_c, &h})
        q->parallelize(k);
    h_init.then(c_init, computation::root)
          .then(h_copy_x, computation::root)
          .then(gates_init, computation::root)
          .then(gates, m)
          .then(sig_i, m)
          .then(sig_f, m)
          .then(tnh_z, m)
          .then(sig_o, m)
          .then(mul_iz, m)
          .then(mul_fc, m)
          .then(c, m)
          .then(tnh_c, m)
          .then(h, m)
          .then(y, computation::root);
    tiramisu::codegen({&buf_weights, &buf_biases, &buf_x, &buf_y}, "build/" + name + "_cpu.o", false);
#else
    for (buffer *q : {&buf_weights, &buf_biases, &buf_x, &buf_y, &buf_gates, &buf_i, &buf_f, &buf_z, &buf_o, &buf_h, &buf_c})
        q->tag_gpu_global();
    var kb("kb"), kt("kt"), ib("ib"), it("it"), gb("gb"), gt("gt"), ls("ls"), ms("ms");
    // fuse the initialisations, the copy of x and the output into one kernel each: layer / time innermost
    for (computation *q : {&h_init, &c_init}) { q->interchange(l, k); q->interchange(l, i); }
    for (computation *q : {&h_copy_x, &y}) { q->interchange(m, k); q->interchange(m, i); }
    // diagonal traversal of (layer, time step); the cells of a diagonal are independent
    block cells({&gates_init, &gates, &sig_i, &sig_f, &tnh_z, &sig_o, &mul_iz, &mul_fc, &c, &tnh_c, &h});
    cells.skew(l, m, 1, ls, ms);
    cells.interchange(ls, ms);
    gates_init.parallelize(ls);
    for (computation *q : {&h_init, &c_init, &h_copy_x, &y, &sig_i, &sig_f, &tnh_z, &sig_o, &mul_iz, &mul_fc, &c, &tnh_c, &h})
        q->gpu_tile(k, i, 16, 16, kb, ib, kt, it);
    gates_init.gpu_tile(k, g, 16, 16, kb, gb, kt, gt);
    gates.gpu_tile(k, g, 16, 16, kb, gb, kt, gt);
    h_init.then(c_init, computation::root)
          .then(h_copy_x, computation::root)
          .then(gates_init, computation::root)
          .then(gates, gt)
          .then(sig_i, ls)
          .then(sig_f, it)
          .then(tnh_z, it)
          .then(sig_o, it)
          .then(mul_iz, it)
          .then(mul_fc, it)
          .then(c, it)
          .then(tnh_c, it)
          .then(h, it)
          .then(y, computation::root);
    tiramisu::codegen({&buf_weights, &buf_biases, &buf_x, &buf_y}, "build/" + name + ".o", true);
#endif
}

int main(int argc, char **argv)
{
    tiramisu::backend_options_from_command_line(argc, argv);
    generate(4, 64, 512, 100);   // benchmark configuration 5
    if (std::getenv("LSTM_ONLY_FULL")) return 0;
    generate(2, 8, 32, 5);
    generate(1, 4, 16, 3);
    generate(3, 20, 64, 4);
    generate(2, 64, 256, 6);     // whole 64x32 tiles with the reduction split over eight groups of wavefronts
    return 0;
}
