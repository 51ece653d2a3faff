// GEMM with a register tile per thread that the reference's own register-tile tests (tests/test_169.cpp -
// test_171.cpp, run unchanged elsewhere in this suite) do not cover: the tile is not square (2 x 6), the grid of
// threads does not divide into whole 16 x 16 thread blocks (48 x 30 threads: the last block row of threads in j
// is partial) and the k range (100) is not a multiple of the k block (32).  A GPU-local accumulator array is
// declared inside the kernel with allocate(), initialised, updated along k (k outermost inside the thread) and
// added to C.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

int main()
{
    const int M = 96, N = 180, K = 100;
    const int RI = 2, RJ = 6, T = 16, KB = 32;
    tiramisu::init("gemm_register_tile");

    var i("i", 0, M), j("j", 0, N), k("k", 0, K);
    var io("io", 0, M / RI), ii("ii", 0, RI), jo("jo", 0, N / RJ), ji("ji", 0, RJ);
    var iob("iob"), iot("iot"), job("job"), jot("jot"), ko("ko"), ki("ki");

    buffer host_A("host_A", {M, K}, p_float32, a_input);
    buffer host_B("host_B", {K, N}, p_float32, a_input);
    buffer host_C("host_C", {M, N}, p_float32, a_output);

    buffer acc_regs("acc_regs", {RI, RJ}, p_float32, a_temporary);
    acc_regs.tag_gpu_local();
    computation acc_decl({io, jo}, allocate(acc_regs));
    computation acc_zero({i, j}, (float)0);

    input A({i, k}, p_float32);
    input B({k, j}, p_float32);
    A.get_buffer()->tag_gpu_global();
    B.get_buffer()->tag_gpu_global();
    computation acc({i, j, k}, p_float32);
    acc.set_expression(acc(i, j, 0) + A(i, k) * B(k, j));
    computation C({i, j}, p_float32);
    C.get_buffer()->tag_gpu_global();
    C.set_expression(C(i, j) + acc(i, j, 0));

    computation up_A({}, memcpy(host_A, *A.get_buffer()));
    computation up_B({}, memcpy(host_B, *B.get_buffer()));
    computation up_C({}, memcpy(host_C, *C.get_buffer()));
    computation down_C({}, memcpy(*C.get_buffer(), host_C));

    acc_decl.gpu_tile(io, jo, T, T, iob, job, iot, jot);
    acc_zero.tile(i, j, RI, RJ, io, jo, ii, ji);
    acc_zero.gpu_tile(io, jo, T, T, iob, job, iot, jot);
    acc.tile(i, j, RI, RJ, io, jo, ii, ji);
    acc.interchange(ji, k);
    acc.interchange(ii, k);
    acc.split(k, KB, ko, ki);
    acc.gpu_tile(io, jo, T, T, iob, job, iot, jot);
    C.tile(i, j, RI, RJ, io, jo, ii, ji);
    C.gpu_tile(io, jo, T, T, iob, job, iot, jot);

    up_A.then(up_B, computation::root)
        .then(up_C, computation::root)
        .then(acc_decl, computation::root)
        .then(acc_zero, jot)
        .then(acc, jot)
        .then(C, jot)
        .then(down_C, computation::root);

    acc_zero.store_in(&acc_regs, {i % RI, j % RJ});
    acc.store_in(&acc_regs, {i % RI, j % RJ});

    tiramisu::codegen({&host_A, &host_B, &host_C}, "build/gemm_register_tile.o", true);
    return 0;
}
