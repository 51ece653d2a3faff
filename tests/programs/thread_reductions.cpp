// Sums whose reduction loop is mapped to GPU threads.  In the reference such a schedule is a data
// race: every thread of the loop does a read-modify-write of the same element (its CUDA printer
// emits the statement as it stands, src/tiramisu_codegen_cuda.cpp:549-707).  The HIP back-end lowers
// it to what the schedule means on a wave64 machine: a private partial sum per thread, a sum across
// the lanes with DPP row shifts and row broadcasts (across wavefronts through LDS when the loop is
// wider than one wavefront) and a single update of the element.
//  * gemv_wavefront        y(i) = sum_j A(i,j) x(j), 300 x 1000: four rows per workgroup, the 64 lanes
//                          of a wavefront share a row (ragged: 1000 = 15 x 64 + 40);
//  * row_sums_quarter_wave s(i) = 1 + sum_j A(i,j), 128 x 50: 16 lanes per row, four rows per wavefront;
//  * row_sums_block        s(i) = sum_j A(i,j), 40 x 5000: 256 threads (four wavefronts) per row;
//  * row_sums_ragged_rows_block  10 x 558, four rows of 256 threads per workgroup: the last workgroup has two rows
//                          only, and its other 512 threads must still reach the barrier of the sum across wavefronts
//                          (the row loop is emitted with a predicate instead of a branch);
//  * row_sums_100_lanes    31 x 450, two rows of 100 threads: the width is rounded up to two wavefronts, the lanes
//                          beyond the loop's extent add zero (and the last workgroup has one row);
//  * row_sums_26_of_64_lanes  80 x 26 split by 64: the thread loop has 26 iterations, the sum runs on 32 lanes;
//  * row_sums_int32_wave, row_sums_int32_block  the same sums on int32 data (50 x 45 on 16 lanes, four rows per
//                          workgroup; 33 x 700 on 128 lanes, two rows per workgroup): the lane shifts move 32-bit
//                          patterns, and a lane without a neighbour adds the all-zero pattern;
//  * row_sums_float64_wave, row_sums_int64_block  64-bit sums (37 x 333 on 32 lanes; 21 x 900 on 192 lanes = three
//                          wavefronts): a value travels between lanes as its two 32-bit halves;
//  * row_sums_uint8_wave, row_sums_int16_block  sums that wrap (45 x 700 uint8 on 64 lanes, 19 x 1300 int16 on 128):
//                          the partial sums are 32-bit, the final store truncates -- the same value modulo 2^8, 2^16;
//  * row_maxima_wave, row_minima_int32_block, row_maxima_int8_wave  m(i) = max (min) over j of A(i, j): the same
//                          lowering with another operation; a lane without a neighbour contributes its identity.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

static void gemv_wavefront()
{
    const int M = 300, N = 1000;
    tiramisu::init("gemv_wavefront");
    var i("i", 0, M), j("j", 0, N), i0("i0"), i1("i1"), j0("j0"), j1("j1");
    input A("A", {i, j}, p_float32);
    input x("x", {j}, p_float32);
    computation y_init("y_init", {i}, expr((float)0));
    computation y("y", {i, j}, p_float32);
    y.store_in(y_init.get_buffer(), {i});
    y.set_expression(y(i, 0) + A(i, j) * x(j));
    y.split(j, 64, j0, j1);
    y.interchange(j0, j1);
    y.split(i, 4, i0, i1);
    y_init.split(i, 4, i0, i1);
#ifndef TIRAMISU_TARGET_CPU
    for (buffer *b : {A.get_buffer(), x.get_buffer(), y_init.get_buffer()}) b->tag_gpu_global();
    y.tag_gpu_block_level(0);
    y.tag_gpu_thread_level(1, 2);            // loops: i0 | i1 j1 | j0
    y_init.tag_gpu_block_level(0);
    y_init.tag_gpu_thread_level(1);
#endif
    y_init.then(y, i1);
#ifdef TIRAMISU_TARGET_CPU
    tiramisu::codegen({A.get_buffer(), x.get_buffer(), y_init.get_buffer()}, "build/gemv_wavefront_cpu.o", false);
#else
    tiramisu::codegen({A.get_buffer(), x.get_buffer(), y_init.get_buffer()}, "build/gemv_wavefront.o", true);
#endif
}

static void row_sums(const std::string &name, int M, int N, int rows_per_block, int lanes, primitive_t type = p_float32)
{
    tiramisu::init(name);
    var i("i", 0, M), j("j", 0, N), i0("i0"), i1("i1"), j0("j0"), j1("j1");
    input A("A", {i, j}, type);
    computation s_init("s_init", {i}, cast(type, expr((float)(rows_per_block > 1 ? 1 : 0))));
    computation s("s", {i, j}, type);
    s.store_in(s_init.get_buffer(), {i});
    s.set_expression(A(i, j) + s(i, 0));     // the element on the right of the sum
    s.split(j, lanes, j0, j1);
    s.interchange(j0, j1);
    s.split(i, rows_per_block, i0, i1);
    s_init.split(i, rows_per_block, i0, i1);
#ifndef TIRAMISU_TARGET_CPU
    for (buffer *b : {A.get_buffer(), s_init.get_buffer()}) b->tag_gpu_global();
    s.tag_gpu_block_level(0);
    s.tag_gpu_thread_level(1, 2);
    s_init.tag_gpu_block_level(0);
    s_init.tag_gpu_thread_level(1);
#endif
    s_init.then(s, i1);
#ifdef TIRAMISU_TARGET_CPU
    tiramisu::codegen({A.get_buffer(), s_init.get_buffer()}, "build/" + name + "_cpu.o", false);
#else
    tiramisu::codegen({A.get_buffer(), s_init.get_buffer()}, "build/" + name + ".o", true);
#endif
}

// the same with a maximum or a minimum instead of the sum: m(i) = max_j A(i, j), starting from A(i, 0)
static void row_extremes(const std::string &name, int M, int N, int rows_per_block, int lanes, primitive_t type, op_t op)
{
    tiramisu::init(name);
    var i("i", 0, M), j("j", 0, N), i0("i0"), i1("i1"), j0("j0"), j1("j1");
    input A("A", {i, j}, type);
    computation m_init("m_init", {i}, A(i, 0));
    computation m("m", {i, j}, type);
    m.store_in(m_init.get_buffer(), {i});
    m.set_expression(expr(op, m(i, 0), A(i, j)));
    m.split(j, lanes, j0, j1);
    m.interchange(j0, j1);
    m.split(i, rows_per_block, i0, i1);
    m_init.split(i, rows_per_block, i0, i1);
#ifndef TIRAMISU_TARGET_CPU
    for (buffer *b : {A.get_buffer(), m_init.get_buffer()}) b->tag_gpu_global();
    m.tag_gpu_block_level(0);
    m.tag_gpu_thread_level(1, 2);
    m_init.tag_gpu_block_level(0);
    m_init.tag_gpu_thread_level(1);
#endif
    m_init.then(m, i1);
#ifdef TIRAMISU_TARGET_CPU
    tiramisu::codegen({A.get_buffer(), m_init.get_buffer()}, "build/" + name + "_cpu.o", false);
#else
    tiramisu::codegen({A.get_buffer(), m_init.get_buffer()}, "build/" + name + ".o", true);
#endif
}

int main()
{
    gemv_wavefront();
    row_sums("row_sums_quarter_wave", 128, 50, 16, 16);
    row_sums("row_sums_block", 40, 5000, 1, 256);
    row_sums("row_sums_ragged_rows_block", 10, 558, 4, 256);
    row_sums("row_sums_100_lanes", 31, 450, 2, 100);
    row_sums("row_sums_26_of_64_lanes", 80, 26, 1, 64);
    row_sums("row_sums_int32_wave", 50, 45, 4, 16, p_int32);
    row_sums("row_sums_int32_block", 33, 700, 2, 128, p_int32);
    row_sums("row_sums_float64_wave", 37, 333, 2, 32, p_float64);
    row_sums("row_sums_int64_block", 21, 900, 2, 192, p_int64);
    row_sums("row_sums_uint8_wave", 45, 700, 1, 64, p_uint8);
    row_sums("row_sums_int16_block", 19, 1300, 2, 128, p_int16);
    row_extremes("row_maxima_wave", 41, 500, 2, 64, p_float32, o_max);
    row_extremes("row_minima_int32_block", 10, 900, 4, 256, p_int32, o_min);
    row_extremes("row_maxima_int8_wave", 30, 333, 4, 16, p_int8, o_max);
    return 0;
}
