// NO_CPU_VARIANT (thread loops run serially on the CPU back-end, which breaks the barrier
// semantics of a cooperative LDS copy; the tests compare with the numpy restatement instead)
// GEMMs whose operand tiles are staged in LDS with cache_shared:
//  * sgemm_shared_regs: alpha * A * B + beta * C in fp32 with a register tile per thread, a local
//    accumulator array declared with allocate(), block-wide scheduling commands, constants read
//    from an input buffer, and both operands cached (A with a padded tile).  Same features as the
//    reference's benchmarks/linear_algebra/blas/level3/sgemm/gpu/generator3.cpp.  Generated twice:
//    sgemm_shared_regs (the back-end proves the LDS tiles and the register tile sound and emits
//    its MFMA kernel) and sgemm_shared_regs_generic (kept as scheduled: cooperative copies,
//    barriers, per-thread array).
//  * gemm_u8_shared: uint8 GEMM (wrap-around arithmetic) with both operands cached, reduction
//    kept in global memory.  Same features as tutorials/developers/tutorial_04gpu2.
#include <cstdlib>
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

static void sgemm_shared_regs(const std::string &name, bool pattern_emitters)
{
    const int M = 256, N = 192, K = 64;
    const int T = 16, KB = 8, RI = 4, RJ = 2;
    tiramisu::init(name);

    var i("i", 0, M), j("j", 0, N), k("k", 0, K);
    var io("io", 0, M / RI), ii("ii", 0, RI), jo("jo", 0, N / RJ), ji("ji", 0, RJ);
    var iob("iob"), iot("iot"), job("job"), jot("jot"), ko("ko"), ki("ki");

    input A({i, k}, p_float32);
    input B({k, j}, p_float32);
    A.get_buffer()->tag_gpu_global();
    B.get_buffer()->tag_gpu_global();
    input scal({i}, p_float32);
    constant alpha("alpha", scal(0));
    constant beta("beta", scal(1));

    computation acc_zero({i, j}, (float)0);
    acc_zero.store_in({i % RI, j % RJ}, {RI, RJ});
    acc_zero.get_buffer()->tag_gpu_local();
    computation acc({i, j, k}, p_float32);
    acc.store_in(acc_zero.get_buffer(), {i % RI, j % RJ});
    acc.set_expression(acc(i, j, 0) + A(i, k) * B(k, j));
    computation C({i, j}, p_float32);
    C.get_buffer()->tag_gpu_global();
    C.set_expression(acc(i, j, 0) * alpha + C(i, j) * beta);
    computation acc_decl({io, jo}, allocate(*acc_zero.get_buffer()));

    buffer host_A("host_A", {M, K}, p_float32, a_input);
    buffer host_B("host_B", {K, N}, p_float32, a_input);
    buffer host_C("host_C", {M, N}, p_float32, a_output);
    computation up_A({}, memcpy(host_A, *A.get_buffer()));
    computation up_B({}, memcpy(host_B, *B.get_buffer()));
    computation up_C({}, memcpy(host_C, *C.get_buffer()));
    computation down_C({}, memcpy(*C.get_buffer(), host_C));

    block({&acc_zero, &acc, &C}).tile(i, j, RI, RJ, io, jo, ii, ji);
    acc.interchange(ji, k);
    acc.interchange(ii, k);
    acc.split(k, KB, ko, ki);
    block kernel({&acc_decl, &acc_zero, &acc, &C});
    kernel.gpu_tile(io, jo, T, T, iob, job, iot, jot);

    up_A.then(up_B)
        .then(up_C)
        .then(acc_decl)
        .then(acc_zero, jot)
        .then(acc, jot)
        .then(C, jot)
        .then(down_C);

    acc.cache_shared(A, ko, {T * RI, KB}, {iob * T * RI, ko * KB}, true);
    acc.cache_shared(B, ko, {KB, T * RJ}, {ko * KB, job * T * RJ});

    if (!pattern_emitters) setenv("TIRAMISU_NO_MFMA", "1", 1);
    tiramisu::codegen({scal.get_buffer(), &host_A, &host_B, &host_C}, "build/" + name + ".o", true);
    if (!pattern_emitters) unsetenv("TIRAMISU_NO_MFMA");
}

static void gemm_u8_shared()
{
    const int S = 128, T = 16, KB = 32;
    tiramisu::init("gemm_u8_shared");
    var i("i", 0, S), j("j", 0, S), k("k", 0, S);
    var ib("ib"), it("it"), jb("jb"), jt("jt"), ko("ko"), ki("ki");

    input A("A", {i, k}, p_uint8);
    input B("B", {k, j}, p_uint8);
    A.get_buffer()->tag_gpu_global();
    B.get_buffer()->tag_gpu_global();
    computation C("C", {i, j, k}, p_uint8);
    C.store_in({i, j}, {S, S});
    C.get_buffer()->tag_gpu_global();
    C.set_expression(C(i, j, 0) + A(i, k) * B(k, j));

    buffer host_A("host_A", {S, S}, p_uint8, a_input);
    buffer host_B("host_B", {S, S}, p_uint8, a_input);
    buffer host_C("host_C", {S, S}, p_uint8, a_output);
    computation up_A({}, memcpy(host_A, *A.get_buffer()));
    computation up_B({}, memcpy(host_B, *B.get_buffer()));
    computation up_C({}, memcpy(host_C, *C.get_buffer()));
    computation down_C({}, memcpy(*C.get_buffer(), host_C));

    C.split(k, KB, ko, ki);
    C.gpu_tile(i, j, T, T, ib, jb, it, jt);
    up_A.then(up_B, computation::root).then(up_C, computation::root).then(C, computation::root).then(down_C, computation::root);

    C.cache_shared(A, ko, {T, KB}, {ib * T, ko * KB});
    C.cache_shared(B, ko, {KB, T}, {ko * KB, jb * T});

    tiramisu::codegen({&host_A, &host_B, &host_C}, "build/gemm_u8_shared.o", true);
}

int main()
{
    sgemm_shared_regs("sgemm_shared_regs", true);
    sgemm_shared_regs("sgemm_shared_regs_generic", false);
    gemm_u8_shared();
    return 0;
}
