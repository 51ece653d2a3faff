// GEMM update kept in global memory: C(i,j) += A(i,k) * B(k,j), the reduction loop split and the
// (i,j) loops mapped to a 16x16 thread grid.  Exercises the same features as the reference's
// tests/test_167.cpp (split + gpu_tile + memcpy + then), on a non-square problem.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

int main(int argc, char **argv)
{
    tiramisu::backend_options_from_command_line(argc, argv);
    const int M = 96, N = 160, K = 64;
    tiramisu::init("gemm_gpu_tile");

    var i("i", 0, M), j("j", 0, N), k("k", 0, K);
    var ib("ib"), it("it"), jb("jb"), jt("jt"), ko("ko"), ki("ki");

    buffer host_A("host_A", {M, K}, p_float32, a_input);
    buffer host_B("host_B", {K, N}, p_float32, a_input);
    buffer host_C("host_C", {M, N}, p_float32, a_output);

    input A({i, k}, p_float32);
    input B({k, j}, p_float32);
    computation C({i, j, k}, p_float32);
    C.store_in({i, j}, {M, N});
    C.set_expression(C(i, j, 0) + A(i, k) * B(k, j));
    A.get_buffer()->tag_gpu_global();
    B.get_buffer()->tag_gpu_global();
    C.get_buffer()->tag_gpu_global();

    computation to_dev_A({}, memcpy(host_A, *A.get_buffer()));
    computation to_dev_B({}, memcpy(host_B, *B.get_buffer()));
    computation to_dev_C({}, memcpy(host_C, *C.get_buffer()));
    computation to_host_C({}, memcpy(*C.get_buffer(), host_C));

    C.split(k, 16, ko, ki);
    C.gpu_tile(i, j, 16, 16, ib, jb, it, jt);

    to_dev_A.then(to_dev_B, computation::root)
            .then(to_dev_C, computation::root)
            .then(C, computation::root)
            .then(to_host_C, computation::root);

    tiramisu::codegen({&host_A, &host_B, &host_C}, "build/gemm_gpu_tile.o", true);
    return 0;
}
