// sgemm: C = alpha * A * B + beta * C, fp32, row-major, as three fused computations -- an
// accumulator initialisation, the k-reduction and the alpha/beta epilogue -- in the style of
// the reference's GPU sgemm generators (benchmarks/linear_algebra/blas/level3/sgemm/gpu/
// generator3.cpp:38-48) with alpha and beta read from an input buffer (:40-42).
//
// GPU schedule: (i, j) tiled 16x16 onto blocks and threads, a one-element register accumulator
// per thread, all three computations fused in the thread; the matrices are GPU-resident
// arguments.  The HIP back-end proves the nest to be a dense contraction and emits its MFMA
// kernel; built with TIRAMISU_NO_MFMA=1 it emits the schedule-faithful kernel instead.
// CPU schedule (-DTIRAMISU_TARGET_CPU): parallelize i, vectorize j by 8, k in between
// (the CPU configuration named by the benchmark description; the reference's tuned variant is
// benchmarks/linear_algebra/blas/level3/sgemm/cpu/sgemm_generator.cpp:127-290).
// One generated function per size: sgemm_<M>x<N>x<K>.
#include <tiramisu/tiramisu.h>

#include <cstdlib>

using namespace tiramisu;

static void generate(int M, int N, int K)
{
    const std::string name = "sgemm_" + std::to_string(M) + "x" + std::to_string(N) + "x" + std::to_string(K);
    tiramisu::init(name);

    var i("i", 0, M), j("j", 0, N), k("k", 0, K), s("s", 0, 2);
    buffer b_scal("b_scal", {2}, p_float32, a_input);
    buffer b_A("b_A", {M, K}, p_float32, a_input);
    buffer b_B("b_B", {K, N}, p_float32, a_input);
    buffer b_C("b_C", {M, N}, p_float32, a_output);

    input scal("scal", {s}, p_float32);
    scal.store_in(&b_scal);
    constant alpha("alpha", scal(0));
    constant beta("beta", scal(1));
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
    var jo("jo"), ji("ji");
    acc.interchange(j, k);
    acc_init.parallelize(i);
    acc.parallelize(i);
    C.parallelize(i);
    if (N % 8 == 0) {
        acc.vectorize(j, 8, jo, ji);
        C.vectorize(j, 8, jo, ji);
    }
    acc_init.then(acc, computation::root).then(C, computation::root);
    tiramisu::codegen({&b_scal, &b_A, &b_B, &b_C}, "build/" + name + "_cpu.o", false);
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
    tiramisu::codegen({&b_scal, &b_A, &b_B, &b_C}, "build/" + name + ".o", true);
#endif
}

int main(int argc, char **argv)
{
    tiramisu::backend_options_from_command_line(argc, argv);
    // SGEMM_ONLY_CUBE=<n>: only the n x n x n instance (for sweeps over the emitter's knobs)
    if (const char *n = std::getenv("SGEMM_ONLY_CUBE")) {
        generate(std::atoi(n), std::atoi(n), std::atoi(n));
        return 0;
    }
    generate(1024, 1024, 1024);   // benchmark configuration 1
    generate(4096, 4096, 4096);   // benchmark configuration 3 (fp32)
    generate(256, 256, 64);
    generate(128, 192, 96);
    generate(100, 70, 50);        // ragged: guarded tile edges
    generate(33, 17, 9);
    generate(64, 256, 512);       // few C tiles, long reduction: wavefront groups split K inside a workgroup
    generate(2048, 2048, 48);     // 256 tiles of 128x128
    generate(3072, 3072, 32);     // 256 tiles of 192x192 (the size of the reference's GPU sgemm benchmark)
    return 0;
}
