// out(i, j) = a(i, j) + 2 a(j, i) for j <= i: a triangular domain under gpu_tile.  After the tiling the bound of the
// block loop over column tiles is a function of the block loop over row tiles (j0 <= (T0 i0 + T0 - 1) / T1) and of
// nothing else: no argument of it is invariant in the kernel, so the launch covers what the bound reaches over the
// range of i0 and a guard in the kernel cuts the triangle out.  (The reference sizes the grid from the loop's own
// upper bound, tiramisu_codegen_cuda.cpp:523-554, which here names an iterator the host does not have.)
//   lower_triangle_16x16: N = 106, tiles 16 x 16;  lower_triangle_16x4: N = 45, tiles 16 x 4 (the bound holds a division)
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

static void lower_triangle(const std::string &name, int N, int T0, int T1)
{
    tiramisu::init(name);
    var i("i", 0, N), j("j", 0, i + 1), i0("i0"), j0("j0"), i1("i1"), j1("j1");
    var ia("ia", 0, N), ja("ja", 0, N);
    input a("a", {ia, ja}, p_int32);
    a.get_buffer()->tag_gpu_global();
    buffer o("o", {N, N}, p_int32, a_output);
    o.tag_gpu_global();
    computation out("out", {i, j}, a(i, j) + a(j, i) * 2);
    out.store_in(&o);
    out.gpu_tile(i, j, T0, T1, i0, j0, i1, j1);
    tiramisu::codegen({a.get_buffer(), &o}, "build/" + name + ".o", true);
}

int main(int argc, char **argv)
{
    tiramisu::backend_options_from_command_line(argc, argv);
    lower_triangle("lower_triangle_16x16", 106, 16, 16);
    lower_triangle("lower_triangle_16x4", 45, 16, 4);
    return 0;
}
