// NO_CPU_VARIANT (on the CPU every statement runs once anyway; the point is what the threads of a workgroup do)
// A kernel whose first statements are under the block loop only:
//   for b (GPU block):
//     weight(b) = 0
//     for k < 5:  weight(b) = weight(b) + (k + 1)          an accumulation that no thread loop encloses
//     for t (GPU thread, 64):  out(b, t) = in(b, t) + weight(b)
// The program means weight(b) = 15.  Every thread of the workgroup reaches the first two statements: emitted as
// they stand (as the reference's CUDA printer would) 64 threads race on the accumulation.  The HIP back-end runs
// statements outside the thread loops on the workgroup's first thread, between barriers.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

// weights_under_conflicting_tags: the same, with the loop level at which the statements are fused tagged differently by
// them -- the weights take (b, c) for (block, thread), the output takes (b, c, u, t) for (block, block, thread, thread),
// as the reference's dibaryon correlators fuse their two-level and four-level statements.  Loop c can be one thing
// only; it is a block dimension, and the weights' statements have no thread loop around them.
static void conflicting_tags()
{
    const int NB = 6, NC = 5, U = 4, T = 16, K = 5;
    tiramisu::init("weights_under_conflicting_tags");
    var b("b", 0, NB), c("c", 0, NC), u("u", 0, U), t("t", 0, T), k("k", 0, K);
    input in("in", {b, c, u, t}, p_float32);
    in.get_buffer()->tag_gpu_global();
    computation weight_init("weight_init", {b, c}, expr(0.0f));
    weight_init.get_buffer()->tag_gpu_global();
    computation weight("weight", {b, c, k}, p_float32);
    weight.store_in(weight_init.get_buffer(), {b, c});
    weight.set_expression(weight(b, c, k - 1) + cast(p_float32, k + 1));
    computation out("out", {b, c, u, t}, in(b, c, u, t) + weight(b, c, K - 1));
    out.get_buffer()->tag_gpu_global();
    weight_init.tag_gpu_level(b, c);
    weight.tag_gpu_level(b, c);
    out.tag_gpu_level(b, c, u, t);
    weight_init.then(weight, c).then(out, c);
    tiramisu::codegen({in.get_buffer(), weight_init.get_buffer(), out.get_buffer()}, "build/weights_under_conflicting_tags.o", true);
}

int main(int argc, char **argv)
{
    tiramisu::backend_options_from_command_line(argc, argv);
    conflicting_tags();
    const int NB = 48, T = 64, K = 5;
    tiramisu::init("weights_outside_thread_loops");
    var b("b", 0, NB), t("t", 0, T), k("k", 0, K);
    input in("in", {b, t}, p_float32);
    in.get_buffer()->tag_gpu_global();
    computation weight_init("weight_init", {b}, expr(0.0f));
    weight_init.get_buffer()->tag_gpu_global();
    computation weight("weight", {b, k}, p_float32);
    weight.store_in(weight_init.get_buffer(), {b});
    weight.set_expression(weight(b, k - 1) + cast(p_float32, k + 1));
    computation out("out", {b, t}, in(b, t) + weight(b, K - 1));
    out.get_buffer()->tag_gpu_global();
    weight_init.tag_gpu_block_level(0);
    weight.tag_gpu_block_level(0);
    out.tag_gpu_level(b, t);
    weight_init.then(weight, b).then(out, b);
    tiramisu::codegen({in.get_buffer(), weight_init.get_buffer(), out.get_buffer()}, "build/weights_outside_thread_loops.o", true);
    return 0;
}
