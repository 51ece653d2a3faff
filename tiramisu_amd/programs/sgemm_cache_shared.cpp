// NO_CPU_VARIANT (the cooperative LDS copy needs its barriers; the CPU back-end runs thread loops serially)
// sgemm with the schedule of the reference's tuned GPU generator
// (benchmarks/linear_algebra/blas/level3/sgemm/gpu/generator3.cpp: 16x16 threads, a 16x8 register
// tile per thread, the reduction split by 4, both operand tiles -- {256, 4} (+1 pad) of A and
// {4, 128} of B -- staged in LDS with cache_shared) at its size, 3072^3, on device-resident buffers,
// KEPT AS SCHEDULED: the pattern emitters are switched off for this function, so the kernel is the
// schedule-faithful emitter's (cooperative copy, two barriers per k-block, per-thread accumulator
// array).  It exists to measure that emitter -- LDS bank conflicts of the padded tiles, coalescing of
// the cooperative copy -- with hardware counters (`python bench.py --workload sgemm_cache_shared`).
#include <cstdlib>
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

int main()
{
    const int M = 3072, N = 3072, K = 3072;
    const int T = 16, KB = 4, RI = 16, RJ = 8;
    tiramisu::init("sgemm_cache_shared_3072");

    var i("i", 0, M), j("j", 0, N), k("k", 0, K);
    var io("io", 0, M / RI), ii("ii", 0, RI), jo("jo", 0, N / RJ), ji("ji", 0, RJ);
    var iob("iob"), iot("iot"), job("job"), jot("jot"), ko("ko"), ki("ki");

    input A("A", {i, k}, p_float32);
    input B("B", {k, j}, p_float32);
    input scal("scal", {i}, p_float32);
    constant alpha("alpha", scal(0));
    constant beta("beta", scal(1));

    computation acc_zero("acc_zero", {i, j}, (float)0);
    acc_zero.store_in({i % RI, j % RJ}, {RI, RJ});
    acc_zero.get_buffer()->tag_gpu_local();
    computation acc("acc", {i, j, k}, p_float32);
    acc.store_in(acc_zero.get_buffer(), {i % RI, j % RJ});
    acc.set_expression(acc(i, j, 0) + A(i, k) * B(k, j));
    computation C("C", {i, j}, p_float32);
    C.set_expression(acc(i, j, 0) * alpha + C(i, j) * beta);
    computation acc_decl("acc_decl", {io, jo}, allocate(*acc_zero.get_buffer()));
    for (buffer *b : {A.get_buffer(), B.get_buffer(), C.get_buffer()}) b->tag_gpu_global();

    block({&acc_zero, &acc, &C}).tile(i, j, RI, RJ, io, jo, ii, ji);
    acc.interchange(ji, k);
    acc.interchange(ii, k);
    acc.split(k, KB, ko, ki);
    block kernel({&acc_decl, &acc_zero, &acc, &C});
    kernel.gpu_tile(io, jo, T, T, iob, job, iot, jot);
    acc_decl.then(acc_zero, jot).then(acc, jot).then(C, jot);

    acc.cache_shared(A, ko, {T * RI, KB}, {iob * T * RI, ko * KB}, true);
    acc.cache_shared(B, ko, {KB, T * RJ}, {ko * KB, job * T * RJ});

    setenv("TIRAMISU_NO_MFMA", "1", 1);      // keep the nest on the schedule-faithful emitter
    tiramisu::codegen({scal.get_buffer(), A.get_buffer(), B.get_buffer(), C.get_buffer()}, "build/sgemm_cache_shared_3072.o", true);
    unsetenv("TIRAMISU_NO_MFMA");
    return 0;
}
