// NO_CPU_VARIANT (the library call only exists in the GPU runtime)
// Row-major GEMM through the GEMM library call with run-time sizes, scalars read from input
// buffers, explicit leading dimensions / element offsets and a transposed operand.  Same
// features as the reference's tests/test_162.cpp and test_164.cpp - test_166.cpp
// (cublas_gemm -> tiramisu_hip_sgemm, constants from inputs, memcpy of argument buffers); the
// second function does the same on doubles (cublas_gemm -> tiramisu_hip_dgemm, what the reference's
// library LSTM uses when its configuration.h is flipped to double precision).
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

// (scalar names are per process: the two functions call theirs differently)
static void library_call(const std::string &name, primitive_t type, const std::string &alpha_name, const std::string &beta_name)
{
    tiramisu::init(name);

    input sizes("sizes", {"si"}, {9}, p_int32);      // M N K ldA ldB ldC offA offB offC
    input scal("scal", {"pi"}, {2}, type);      // alpha beta
    constant M("M", sizes(0)), N("N", sizes(1)), K("K", sizes(2));
    constant ldA("ldA", sizes(3)), ldB("ldB", sizes(4)), ldC("ldC", sizes(5));
    constant offA("offA", sizes(6)), offB("offB", sizes(7)), offC("offC", sizes(8));
    constant alpha(alpha_name, scal(0)), beta(beta_name, scal(1));

    // A is stored transposed (K rows of ldA elements), B and C plain.
    input A("A", {"a0", "a1"}, {K + 1, ldA}, type);
    input B("B", {"b0", "b1"}, {K + 1, ldB}, type);
    input C("C", {"c0", "c1"}, {M + 1, ldC}, type);

    buffer dA("dA", {K + 1, ldA}, type, a_temporary);
    buffer dB("dB", {K + 1, ldB}, type, a_temporary);
    buffer dC("dC", {M + 1, ldC}, type, a_temporary);
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
                      "build/" + name + ".o", true);
}

int main()
{
    library_call("sgemm_library_call", p_float32, "alpha", "beta");
    library_call("dgemm_library_call", p_float64, "alpha_d", "beta_d");
    return 0;
}
