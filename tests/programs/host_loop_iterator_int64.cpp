// NO_CPU_VARIANT (the point is the kernel's parameter list on the HIP back-end; checked against numpy)
// Kernels launched inside a host loop whose iterator they use, in a program that sets the loop iterator type to
// 64 bits (global::set_loop_iterator_type(p_int64), as the reference's tensor-contraction benchmarks do): the
// generated host loops are int32_t all the same, and the launch hands the kernel the address of that variable --
// a kernel that declared the parameter with the program's 64-bit type would read past it.
//   planes(p, i, j) = in(i, j) * (p + 1) + p           p is a host loop around the kernel
// Generated twice: host_loop_iterator_int64 with the loop serial (the iterator is a kernel parameter) and
// host_loop_iterator_int64_parallel with the loop tagged parallel (its iterations become gridDim.z and the
// first one a kernel parameter).
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

static void generate(const std::string &name, bool parallel)
{
    const int P = 5, N = 128;
    tiramisu::init(name);
    global::set_loop_iterator_type(p_int64);

    var p("p", 0, P), i("i", 0, N), j("j", 0, N);
    var ib("ib"), jb("jb"), it("it"), jt("jt");
    buffer b_in("b_in", {N, N}, p_float32, a_input);
    buffer b_planes("b_planes", {P, N, N}, p_float32, a_output);
    b_in.tag_gpu_global();
    b_planes.tag_gpu_global();
    input in("in", {i, j}, p_float32);
    in.store_in(&b_in);
    computation planes("planes", {p, i, j}, in(i, j) * cast(p_float32, p + 1) + cast(p_float32, p));
    planes.store_in(&b_planes);
    planes.gpu_tile(i, j, 16, 16, ib, jb, it, jt);
    if (parallel) planes.tag_parallel_level(p);
    tiramisu::codegen({&b_in, &b_planes}, "build/" + name + ".o", true);
    global::set_loop_iterator_type(p_int32);
}

int main(int argc, char **argv)
{
    tiramisu::backend_options_from_command_line(argc, argv);
    generate("host_loop_iterator_int64", false);
    generate("host_loop_iterator_int64_parallel", true);
    return 0;
}
