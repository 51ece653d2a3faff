// NO_CPU_VARIANT (the point is what the generator says about the GPU code; nothing here is run)
// Sums on GPU threads that the back-end does not lower, and says so on stderr instead of emitting the race silently:
//  * row_sums_bf16: s(i) = sum_j A(i, j) stored as bfloat16 on 64 lanes (sums of integers, float and double are lowered);
//  * update_inside_one_thread_loop_only: two rows per workgroup, the row sum on 16 lanes (lowered), and beside its
//    initialisation a statement bump(i): s(i) = s(i) + 2 that lies inside the loop over rows (threadIdx.y) but outside
//    the loop over lanes (threadIdx.x): all 16 lanes of a row execute it;
//  * row_sums_of_even_columns: the row sum on 64 lanes with a predicate on the statement (j % 2 == 0);
//  * tile_sums: s(b) = sum over y, x of A(b, y, x) with both y and x mapped to threads.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

static void row_sums_bf16()
{
    const int M = 20, N = 300;
    tiramisu::init("row_sums_bf16");
    var i("i", 0, M), j("j", 0, N), j0("j0"), j1("j1");
    input A("A", {i, j}, p_bfloat16);
    computation s_init("s_init", {i}, cast(p_bfloat16, expr((float)0)));
    computation s("s", {i, j}, p_bfloat16);
    s.store_in(s_init.get_buffer(), {i});
    s.set_expression(A(i, j) + s(i, 0));
    s.split(j, 64, j0, j1);
    s.interchange(j0, j1);
    for (buffer *b : {A.get_buffer(), s_init.get_buffer()}) b->tag_gpu_global();
    s.tag_gpu_block_level(0);
    s.tag_gpu_thread_level(1);
    s_init.tag_gpu_block_level(0);
    s_init.then(s, 0);
    tiramisu::codegen({A.get_buffer(), s_init.get_buffer()}, "build/row_sums_bf16.o", true);
}

static void update_inside_one_thread_loop_only()
{
    const int M = 20, N = 300;
    tiramisu::init("update_inside_one_thread_loop_only");
    var i("i", 0, M), j("j", 0, N), i0("i0"), i1("i1"), j0("j0"), j1("j1");
    input A("A", {i, j}, p_float32);
    computation s_init("s_init", {i}, expr((float)0));
    computation bump("bump", {i}, p_float32);
    bump.store_in(s_init.get_buffer(), {i});
    bump.set_expression(s_init(i) + expr((float)2));
    computation s("s", {i, j}, p_float32);
    s.store_in(s_init.get_buffer(), {i});
    s.set_expression(A(i, j) + s(i, 0));
    s.split(j, 16, j0, j1);
    s.interchange(j0, j1);
    s.split(i, 2, i0, i1);
    s_init.split(i, 2, i0, i1);
    bump.split(i, 2, i0, i1);
    for (buffer *b : {A.get_buffer(), s_init.get_buffer()}) b->tag_gpu_global();
    s.tag_gpu_block_level(0);
    s.tag_gpu_thread_level(1, 2);
    for (computation *c : {&s_init, &bump}) {
        c->tag_gpu_block_level(0);
        c->tag_gpu_thread_level(1);
    }
    s_init.then(bump, i1).then(s, i1);
    tiramisu::codegen({A.get_buffer(), s_init.get_buffer()}, "build/update_inside_one_thread_loop_only.o", true);
}

static void row_sums_of_even_columns()
{
    const int M = 20, N = 300;
    tiramisu::init("row_sums_of_even_columns");
    var i("i", 0, M), j("j", 0, N), j0("j0"), j1("j1");
    input A("A", {i, j}, p_float32);
    computation s_init("s_init", {i}, expr((float)0));
    computation s("s", {i, j}, p_float32);
    s.store_in(s_init.get_buffer(), {i});
    s.set_expression(A(i, j) + s(i, 0));
    s.add_predicate(j % 2 == 0);
    s.split(j, 64, j0, j1);
    s.interchange(j0, j1);
    for (buffer *b : {A.get_buffer(), s_init.get_buffer()}) b->tag_gpu_global();
    s.tag_gpu_block_level(0);
    s.tag_gpu_thread_level(1);
    s_init.tag_gpu_block_level(0);
    s_init.then(s, 0);
    tiramisu::codegen({A.get_buffer(), s_init.get_buffer()}, "build/row_sums_of_even_columns.o", true);
}

static void tile_sums()
{
    tiramisu::init("tile_sums");
    var b("b", 0, 30), y("y", 0, 8), x("x", 0, 16);
    input A("A", {b, y, x}, p_float32);
    computation s_init("s_init", {b}, expr((float)0));
    computation s("s", {b, y, x}, p_float32);
    s.store_in(s_init.get_buffer(), {b});
    s.set_expression(A(b, y, x) + s(b, 0, 0));
    for (buffer *buf : {A.get_buffer(), s_init.get_buffer()}) buf->tag_gpu_global();
    s.tag_gpu_block_level(0);
    s.tag_gpu_thread_level(1, 2);
    s_init.tag_gpu_block_level(0);
    s_init.then(s, 0);
    tiramisu::codegen({A.get_buffer(), s_init.get_buffer()}, "build/tile_sums.o", true);
}

int main(int argc, char **argv)
{
    tiramisu::backend_options_from_command_line(argc, argv);
    row_sums_bf16();
    update_inside_one_thread_loop_only();
    row_sums_of_even_columns();
    tile_sums();
    return 0;
}
