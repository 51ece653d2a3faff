// sgemm whose sizes are run-time values: M, N, K come from an input buffer, as in the reference's
// GPU sgemm generators (benchmarks/linear_algebra/blas/level3/sgemm/gpu/generator3.cpp:27-42 reads
// SIZES and alpha/beta from buffers).  Loop bounds, buffer extents, grid sizes and tile-edge guards
// are then symbolic in the generated code; one compiled function serves every size, including
// ragged and empty ones.  The matrices are GPU-resident arguments.  Two functions are generated:
// sgemm_runtime_sizes (the back-end recognises the contraction) and sgemm_runtime_sizes_generic
// (pattern emitters switched off: the schedule-faithful kernel, one thread per (i, j)).
#include <cstdlib>
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

static void generate(const std::string &name, bool pattern_emitters)
{
    tiramisu::init(name);

    var d("d", 0, 3), s("s", 0, 2);
    buffer b_sizes("b_sizes", {3}, p_int32, a_input);
    buffer b_scal("b_scal", {2}, p_float32, a_input);
    input sizes("sizes", {d}, p_int32);
    input scal("scal", {s}, p_float32);
    sizes.store_in(&b_sizes);
    scal.store_in(&b_scal);
    constant M("M", sizes(0)), N("N", sizes(1)), K("K", sizes(2));
    constant alpha("alpha", scal(0)), beta("beta", scal(1));

    var i("i", 0, M), j("j", 0, N), k("k", 0, K);
    buffer b_A("b_A", {M, K}, p_float32, a_input);
    buffer b_B("b_B", {K, N}, p_float32, a_input);
    buffer b_C("b_C", {M, N}, p_float32, a_output);
    input A("A", {i, k}, p_float32);
    input B("B", {k, j}, p_float32);
    A.store_in(&b_A);
    B.store_in(&b_B);

    computation acc_init("acc_init", {i, j}, expr((float)0));
    computation acc("acc", {i, j, k}, p_float32);
    acc.set_expression(acc(i, j, 0) + A(i, k) * B(k, j));
    computation C("C", {i, j}, p_float32);
    C.set_expression(acc(i, j, 0) * alpha + C(i, j) * beta);
    C.store_in(&b_C);

#ifdef TIRAMISU_TARGET_CPU
    buffer b_acc("b_acc", {M, N}, p_float32, a_temporary);
    acc_init.store_in(&b_acc, {i, j});
    acc.store_in(&b_acc, {i, j});
    acc_init.then(acc, computation::root).then(C, computation::root);
    (void)pattern_emitters;
    tiramisu::codegen({&b_sizes, &b_scal, &b_A, &b_B, &b_C}, "build/" + name + "_cpu.o", false);
#else
    b_A.tag_gpu_global();
    b_B.tag_gpu_global();
    b_C.tag_gpu_global();
    buffer acc_reg("acc_reg", {1}, p_float32, a_temporary);
    acc_reg.tag_gpu_register();
    computation acc_decl("acc_decl", {i, j}, allocate(acc_reg));
    acc_init.store_in(&acc_reg, {0});
    acc.store_in(&acc_reg, {0});
    var ib("ib"), jb("jb"), it("it"), jt("jt");
    block({&acc_decl, &acc_init, &acc, &C}).gpu_tile(i, j, 16, 16, ib, jb, it, jt);
    acc_decl.then(acc_init, jt).then(acc, jt).then(C, jt);
    if (!pattern_emitters) setenv("TIRAMISU_NO_MFMA", "1", 1);
    tiramisu::codegen({&b_sizes, &b_scal, &b_A, &b_B, &b_C}, "build/" + name + ".o", true);
    if (!pattern_emitters) unsetenv("TIRAMISU_NO_MFMA");
#endif
}

int main()
{
    generate("sgemm_runtime_sizes", true);
    generate("sgemm_runtime_sizes_generic", false);
    return 0;
}
