// A sum over a loop of 256 GPU threads that sits under a condition: rows 3 .. 39 of s(i) = sum_j A(i, j) are summed,
// rows 0 .. 2 only initialised, both statements in one block loop -- so the generated kernel tests the block
// iterator before the thread loop.  The lowering of such a sum across wavefronts ends in a workgroup barrier,
// which every thread must reach: a condition on block iterators alone is the same for the whole workgroup, so the
// sum is lowered below it (a condition that names a thread iterator would keep the loop as the program states it).
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

int main()
{
    const int M = 40, N = 5000;
    tiramisu::init("row_sums_from_row_3");
    var i("i", 0, M), iu("iu", 3, M), j("j", 0, N), j0("j0"), j1("j1");
    input A("A", {i, j}, p_float32);
    computation s_init("s_init", {i}, expr((float)0));
    computation s("s", {iu, j}, p_float32);
    s.store_in(s_init.get_buffer(), {iu});
    s.set_expression(A(iu, j) + s(iu, 0));
    s.split(j, 256, j0, j1);
    s.interchange(j0, j1);
    for (buffer *b : {A.get_buffer(), s_init.get_buffer()}) b->tag_gpu_global();
    s.tag_gpu_block_level(0);
    s.tag_gpu_thread_level(1);
    s_init.tag_gpu_block_level(0);
    s_init.then(s, 0);
    tiramisu::codegen({A.get_buffer(), s_init.get_buffer()}, "build/row_sums_from_row_3.o", true);
    return 0;
}
