// NO_CPU_VARIANT (the point is the host-side threading of the HIP back-end; checked against numpy)
// A host loop tagged parallel around GPU kernels, as the reference's library LSTM has it
// (benchmarks/DNN/blocks/LSTM/gpu_lib/generator.cpp:133-135): the iterations of p run on pool
// threads, each on a stream of its own.
//   base(i, j)    = in(i, j) + 1                          one kernel before the loop
//   for p (parallel):
//     s1(p, i, j) = base(i, j) * (p + 1)                  kernel
//     s2(p, i, j) = s1(p, i, j) + s1(p, N - 1 - i, j)     kernel; reads rows other threads of the first wrote
//   out(i, j)     = sum over p of s2(p, i, j)             one kernel after the loop
// More iterations (6) than pool threads; what runs before the loop must be complete when the first
// iteration starts, the two kernels of an iteration must stay in order, and the last kernel
// must see every iteration's result.  Generated three times: parallel_host_loop (the pool: the distribution of
// the loop over its statements is switched off through a back-end option), parallel_host_loop_distributed (what the
// back-end does when left alone: each of the two kernels once, with the six iterations as gridDim.z), and
// parallel_host_loop_serial with the tag ignored.
#include <cstdlib>
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

enum how_t { pool, distributed, serial };

static void generate(const std::string &name, how_t how)
{
    const int P = 6, N = 256;
    tiramisu::init(name);

    var p("p", 0, P), i("i", 0, N), j("j", 0, N);
    var ib("ib"), jb("jb"), it("it"), jt("jt");

    buffer b_in("b_in", {N, N}, p_float32, a_input);
    buffer b_base("b_base", {N, N}, p_float32, a_temporary);
    buffer b_s1("b_s1", {P, N, N}, p_float32, a_temporary);
    buffer b_s2("b_s2", {P, N, N}, p_float32, a_temporary);
    buffer b_out("b_out", {N, N}, p_float32, a_output);
    for (buffer *b : {&b_in, &b_base, &b_s1, &b_s2, &b_out}) b->tag_gpu_global();

    input in("in", {i, j}, p_float32);
    in.store_in(&b_in);
    computation base("base", {i, j}, in(i, j) + 1.0f);
    base.store_in(&b_base);
    computation s1("s1", {p, i, j}, base(i, j) * cast(p_float32, p + 1));
    s1.store_in(&b_s1);
    computation s2("s2", {p, i, j}, p_float32);
    s2.set_expression(s1(p, i, j) + s1(p, N - 1 - i, j));
    s2.store_in(&b_s2);
    computation out_init("out_init", {i, j}, expr(0.0f));
    out_init.store_in(&b_out, {i, j});
    computation out("out", {i, j, p}, p_float32);
    out.set_expression(out(i, j, 0) + s2(p, i, j));
    out.store_in(&b_out, {i, j});

    base.gpu_tile(i, j, 16, 16, ib, jb, it, jt);
    s1.gpu_tile(i, j, 16, 16, ib, jb, it, jt);
    s2.gpu_tile(i, j, 16, 16, ib, jb, it, jt);
    block({&out_init, &out}).gpu_tile(i, j, 16, 16, ib, jb, it, jt);
    s1.tag_parallel_level(p);
    base.then(s1, computation::root).then(s2, p).then(out_init, computation::root).then(out, jt);

    if (how == serial) tiramisu::set_backend_option("hip_serial_host_loops", "1");
    if (how == pool) tiramisu::set_backend_option("hip_no_distributed_host_loops", "1");
    tiramisu::codegen({&b_in, &b_out}, "build/" + name + ".o", true);
}

int main()
{
    generate("parallel_host_loop", pool);
    generate("parallel_host_loop_distributed", distributed);
    generate("parallel_host_loop_serial", serial);
    return 0;
}
