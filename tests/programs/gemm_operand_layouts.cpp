// C(i,j) += X * Y with the operands stored in each of the four layouts -- A as [M][K] or [K][M], B as
// [K][N] or [N][K] -- and, in a fifth function, inside larger buffers (row pitch and origin that are
// not multiples of 4 elements).  All five nests are dense contractions for the MFMA emitter; its
// operand analysis decides per operand whether k or the row index is the contiguous direction and
// whether 16-byte loads are allowed.  One function per case: gemm_layout_<nn|nt|tn|tt|pitched>.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

static void generate(const std::string &tag, bool a_transposed, bool b_transposed, int pad, int origin)
{
    const int M = 96, N = 80, K = 72;
    tiramisu::init("gemm_layout_" + tag);

    var i("i", 0, M), j("j", 0, N), k("k", 0, K);
    var ib("ib"), it("it"), jb("jb"), jt("jt");

    const int a_rows = a_transposed ? K : M, a_cols = a_transposed ? M : K;
    const int b_rows = b_transposed ? N : K, b_cols = b_transposed ? K : N;
    buffer buf_A("buf_A", {a_rows + origin, a_cols + pad}, p_float32, a_input);
    buffer buf_B("buf_B", {b_rows + origin, b_cols + pad}, p_float32, a_input);
    buffer buf_C("buf_C", {M, N}, p_float32, a_output);
    for (buffer *b : {&buf_A, &buf_B, &buf_C}) b->tag_gpu_global();

    input A("A", {i, k}, p_float32);
    input B("B", {k, j}, p_float32);
    if (a_transposed) A.store_in(&buf_A, {k + origin, i + (pad ? 1 : 0)});
    else A.store_in(&buf_A, {i + origin, k + (pad ? 1 : 0)});
    if (b_transposed) B.store_in(&buf_B, {j + origin, k + (pad ? 1 : 0)});
    else B.store_in(&buf_B, {k + origin, j + (pad ? 1 : 0)});

    computation C("C", {i, j, k}, p_float32);
    C.set_expression(C(i, j, 0) + A(i, k) * B(k, j));
    C.store_in(&buf_C, {i, j});
    C.gpu_tile(i, j, 16, 16, ib, jb, it, jt);

    tiramisu::codegen({&buf_A, &buf_B, &buf_C}, "build/gemm_layout_" + tag + ".o", true);
}

int main()
{
    generate("nn", false, false, 0, 0);
    generate("nt", false, true, 0, 0);
    generate("tn", true, false, 0, 0);
    generate("tt", true, true, 0, 0);
    generate("pitched", false, true, 3, 2);
    return 0;
}
