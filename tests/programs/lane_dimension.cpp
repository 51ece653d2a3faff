// Which tagged thread loop runs along the lanes of a wavefront.
//  * lanes_follow_unit_stride   out(x, y) = 2 in(x, y) + in(x + 1, y) on buffers laid out [y][x], tiled
//                               gpu_tile(x, y, 16, 16): the innermost tagged loop is y, which the reference's
//                               numbering (x, y, z from the innermost tagged level outwards,
//                               src/tiramisu_codegen_cuda.cpp:560-617) would put on threadIdx.x although every
//                               access has unit stride along x -- the layout of the image pipelines under
//                               benchmarks/halide.  150 x 70: ragged tiles.
//  * column_sums_keep_lanes     s(i) = sum_j A(j, i): the loop over j is mapped to the 64 lanes (a sum across
//                               threads) while the loads have unit stride along i; the numbering stays, because
//                               the lowering of the sum is tied to threadIdx.x.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

static void lanes_follow_unit_stride()
{
    const int W = 150, H = 70;
    tiramisu::init("lanes_follow_unit_stride");
    var x("x", 0, W), y("y", 0, H), xe("xe", 0, W + 1), x0("x0"), y0("y0"), x1("x1"), y1("y1");
    buffer b_in("b_in", {H, W + 1}, p_float32, a_input);
    buffer b_out("b_out", {H, W}, p_float32, a_output);
    input in("in", {xe, y}, p_float32);
    in.store_in(&b_in, {y, xe});
    computation out("out", {x, y}, in(x, y) * expr(2.0f) + in(x + 1, y));
    out.store_in(&b_out, {y, x});
#ifndef TIRAMISU_TARGET_CPU
    b_in.tag_gpu_global();
    b_out.tag_gpu_global();
    out.gpu_tile(x, y, 16, 16, x0, y0, x1, y1);
    tiramisu::codegen({&b_in, &b_out}, "build/lanes_follow_unit_stride.o", true);
#else
    tiramisu::codegen({&b_in, &b_out}, "build/lanes_follow_unit_stride_cpu.o", false);
#endif
}

static void column_sums_keep_lanes()
{
    const int M = 96, N = 192;               // columns, rows
    tiramisu::init("column_sums_keep_lanes");
    var i("i", 0, M), j("j", 0, N), i0("i0"), i1("i1"), j0("j0"), j1("j1");
    buffer b_A("b_A", {N, M}, p_float32, a_input);
    input A("A", {j, i}, p_float32);
    A.store_in(&b_A, {j, i});
    computation s_init("s_init", {i}, expr((float)0));
    computation s("s", {i, j}, p_float32);
    s.store_in(s_init.get_buffer(), {i});
    s.set_expression(s(i, 0) + A(j, i));
    s.split(j, 64, j0, j1);
    s.interchange(j0, j1);
    s.split(i, 4, i0, i1);
    s_init.split(i, 4, i0, i1);
#ifndef TIRAMISU_TARGET_CPU
    b_A.tag_gpu_global();
    s_init.get_buffer()->tag_gpu_global();
    s.tag_gpu_block_level(0);
    s.tag_gpu_thread_level(1, 2);            // loops: i0 | i1 j1 | j0
    s_init.tag_gpu_block_level(0);
    s_init.tag_gpu_thread_level(1);
#endif
    s_init.then(s, i1);
#ifdef TIRAMISU_TARGET_CPU
    tiramisu::codegen({&b_A, s_init.get_buffer()}, "build/column_sums_keep_lanes_cpu.o", false);
#else
    tiramisu::codegen({&b_A, s_init.get_buffer()}, "build/column_sums_keep_lanes.o", true);
#endif
}

int main()
{
    lanes_follow_unit_stride();
    column_sums_keep_lanes();
    return 0;
}
