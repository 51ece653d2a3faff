// sgemm with bf16 inputs and fp32 accumulation: C = alpha * A * B + beta * C where A and B are
// stored as bfloat16 and every product and sum is carried out in fp32 (the bf16-input variant of
// benchmark configuration 3).  The reference has no 16-bit float type (include/tiramisu/type.h:27-44);
// this build adds p_bfloat16 as a storage type: a read widens to fp32, arithmetic is fp32.
// Same computation structure and schedules as sgemm.cpp.  One generated function per size:
// sgemm_bf16_<M>x<N>x<K>.
#include <tiramisu/tiramisu.h>

#include <cstdlib>

using namespace tiramisu;

static void generate(int M, int N, int K)
{
    const std::string name = "sgemm_bf16_" + std::to_string(M) + "x" + std::to_string(N) + "x" + std::to_string(K);
    tiramisu::init(name);

    var i("i", 0, M), j("j", 0, N), k("k", 0, K), s("s", 0, 2);
    buffer b_scal("b_scal", {2}, p_float32, a_input);
    buffer b_A("b_A", {M, K}, p_bfloat16, a_input);
    buffer b_B("b_B", {K, N}, p_bfloat16, a_input);
    buffer b_C("b_C", {M, N}, p_float32, a_output);

    input scal("scal", {s}, p_float32);
    scal.store_in(&b_scal);
    constant alpha("alpha", scal(0));
    constant beta("beta", scal(1));
    input A("A", {i, k}, p_bfloat16);
    input B("B", {k, j}, p_bfloat16);
    A.store_in(&b_A);
    B.store_in(&b_B);

    computation acc_init("acc_init", {i, j}, expr((float)0));
    computation acc("acc", {i, j, k}, p_float32);
    acc.set_expression(acc(i, j, 0) + cast(p_float32, A(i, k)) * cast(p_float32, B(k, j)));
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
    generate(4096, 4096, 4096);   // benchmark configuration 3, bf16-input variant
    if (std::getenv("SGEMM_BF16_ONLY_FULL")) return 0;   // for sweeps over the emitter's knobs
    generate(4096, 3072, 32);     // 256x256 tiles, a single K-slice
    generate(3072, 4096, 160);    // 256x256 tiles, five K-slices: one steady-state turn of the four-stage ring, then the drain
    generate(1024, 1280, 512);    // 128x128 tiles
    generate(128, 192, 128);      // whole 64x64x64 tiles: MFMA path
    generate(48, 40, 24);         // one ragged 64x64 tile: MFMA path with guarded loads
    generate(200, 150, 100);      // ragged in every direction, rows of neither operand 16-byte aligned
    return 0;
}
