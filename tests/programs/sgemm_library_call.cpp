// NO_CPU_VARIANT (the library call only exists in the GPU runtime)
// Row-major SGEMM through the GEMM library call with run-time sizes, scalars read from input
// buffers, explicit leading dimensions / element offsets and a transposed operand.  Same
// features as the reference's tests/test_162.cpp and test_164.cpp - test_166.cpp
// (cublas_gemm -> tiramisu_hip_sgemm, constants from inputs, memcpy of argument buffers).
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

int main()
{
    tiramisu::init("sgemm_library_call");

    input sizes("sizes", {"si"}, {9}, p_int32);      // M N K ldA ldB ldC offA offB offC
    input scal("scal", {"pi"}, {2}, p_float32);      // alpha beta
    constant M("M", sizes(0)), N("N", sizes(1)), K("K", sizes(2));
    constant ldA("ldA", sizes(3)), ldB("ldB", sizes(4)), ldC("ldC", sizes(5));
    constant offA("offA", sizes(6)), offB("offB", sizes(7)), offC("offC", sizes(8));
    constant alpha("alpha", scal(0)), beta("beta", scal(1));

    // A is stored transposed (K rows of ldA elements), B and C plain.
    input A("A", {"a0", "a1"}, {K + 1, ldA}, p_float32);
    input B("B", {"b0", "b1"}, {K + 1, ldB}, p_float32);
    input C("C", {"c0", "c1"}, {M + 1, ldC}, p_float32);

    buffer dA("dA", {K + 1, ldA}, p_float32, a_temporary);
    buffer dB("dB", {K + 1, ldB}, p_float32, a_temporary);
    buffer dC("dC", {M + 1, ldC}, p_float32, a_temporary);
    dA.tag_gpu_global();
    dB.tag_gpu_global();
    dC.tag_gpu_global();

    computation up_A({}, memcpy(*A.get_buffer(), dA));
    computation up_B({}, memcpy(*B.get_buffer(), dB));
    computation up_C({}, memcpy(*C.get_buffer(), dC));
    computation gemm({var("once", 0, 1)},
                     cublas_gemm(dA, dB, dC, M, N, K, alpha, beta, ldA, ldB, ldC, offA, offB, offC,
                                 value_cast(p_boolean, 1), value_cast(p_boolean, 0)));
    computation down_C({}, memcpy(dC, *C.get_buffer()));

    up_A.then(up_B, computation::root)
        .then(up_C, computation::root)
        .then(gemm, computation::root)
        .then(down_C, computation::root);

    tiramisu::codegen({sizes.get_buffer(), scal.get_buffer(), A.get_buffer(), B.get_buffer(), C.get_buffer()},
                      "build/sgemm_library_call.o", true);
    return 0;
}
