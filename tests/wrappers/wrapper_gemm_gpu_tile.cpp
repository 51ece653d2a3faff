// C++ wrapper of the generated function gemm_gpu_tile (tests/programs/gemm_gpu_tile.cpp), written
// the way the reference's wrappers are (tests/wrapper_test_167.cpp:6-33 of the reference tree):
// Halide::Buffer arguments, a nested-loop reference, compare_buffers.  Exit status 0 on success.
// links: tests/programs/build/gemm_gpu_tile.o
#include "Halide.h"
#include <tiramisu/utils.h>

#include <cstdlib>

extern "C" int gemm_gpu_tile(halide_buffer_t *A, halide_buffer_t *B, halide_buffer_t *C);

int main(int, char **)
{
    const int M = 96, K = 64, N = 160;
    // extents innermost first: A is M rows of K, B is K rows of N, C is M rows of N
    Halide::Buffer<float> A(K, M), B(N, K), C(N, M), C_ref(N, M);
    std::srand(167);
    for (int m = 0; m < M; m++)
        for (int k = 0; k < K; k++) A(k, m) = (float)(std::rand() % 10 - 5);
    for (int k = 0; k < K; k++)
        for (int n = 0; n < N; n++) B(n, k) = (float)(std::rand() % 10 - 5);
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) C(n, m) = (float)(std::rand() % 10 - 5);
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) {
            float acc = C(n, m);
            for (int k = 0; k < K; k++) acc += A(k, m) * B(n, k);
            C_ref(n, m) = acc;
        }

    gemm_gpu_tile(A.raw_buffer(), B.raw_buffer(), C.raw_buffer());
    compare_buffers("gemm_gpu_tile", C, C_ref);
    return 0;
}
