// NO_CPU_VARIANT (only the kind of kernel that the HIP back-end chooses is looked at; see below)
// What the back-end must prove before it replaces a scheduled GEMM nest by its MFMA kernel, on
// the schedule of the reference's benchmarks/linear_algebra/blas/level3/sgemm/gpu/generator3.cpp
// (register tile per thread below the split reduction loop, both operands through cache_shared):
//  * proofs_sound:           the schedule as the reference writes it       -> MFMA kernel
//  * proofs_short_tile:      the LDS tile of A holds half the k range that
//                            an iteration of the copy level reads          -> kept as scheduled
//  * proofs_shifted_tile:    the LDS tile of B starts one tile to the right -> kept as scheduled
//  * proofs_unaligned_tile:  tile origin not a multiple of the tile shape
//                            (the redirected load indexes modulo the shape) -> kept as scheduled
//  * proofs_shared_register: two rows of a thread's register tile share
//                            one accumulator element                       -> kept as scheduled
//  * proofs_epilogue_other_element: a plain nest (global accumulator, one
//                            thread per row) whose fused epilogue reads the
//                            accumulator of column 0, not its own element   -> kept as scheduled
// The four flawed tilings compute something else than the GEMM when run as scheduled (and the
// shifted tile reads past its operand), so they are generated and inspected, never run.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

enum flaw { none, short_tile, shifted_tile, unaligned_tile, shared_register };

static void generate(const std::string &name, flaw what)
{
    const int M = 256, N = 256, K = 128;
    const int T = 8, KB = 8, RI = 4, RJ = 4;
    tiramisu::init(name);

    var i("i", 0, M), j("j", 0, N), k("k", 0, K);
    var i0("i0", 0, M / RI), i1("i1", 0, RI), j0("j0", 0, N / RJ), j1("j1", 0, RJ);
    var i00("i00"), i01("i01"), j00("j00"), j01("j01"), k0("k0"), k1("k1");

    input A({i, k}, p_float32);
    input B({k, j}, p_float32);
    A.get_buffer()->tag_gpu_global();
    B.get_buffer()->tag_gpu_global();

    const int rows = what == shared_register ? RI / 2 : RI;
    computation acc_init({i, j}, (float)0);
    acc_init.store_in({i % rows, j % RJ}, {rows, RJ});
    acc_init.get_buffer()->tag_gpu_local();
    computation acc({i, j, k}, p_float32);
    acc.store_in(acc_init.get_buffer(), {i % rows, j % RJ});
    acc.set_expression(acc(i, j, 0) + A(i, k) * B(k, j));
    computation C({i, j}, p_float32);
    C.get_buffer()->tag_gpu_global();
    C.set_expression(acc(i, j, 0) + C(i, j));
    computation acc_dec({i0, j0}, allocate(*acc_init.get_buffer()));

    block({&acc_init, &acc, &C}).tile(i, j, RI, RJ, i0, j0, i1, j1);
    acc.interchange(j1, k);
    acc.interchange(i1, k);
    acc.split(k, KB, k0, k1);
    block({&acc_dec, &acc_init, &acc, &C}).gpu_tile(i0, j0, T, T, i00, j00, i01, j01);
    acc_dec.then(acc_init, j01).then(acc, j01).then(C, j01);

    const int kshape = what == short_tile ? KB / 2 : KB;
    expr a_row = i00 * T * RI, b_col = j00 * T * RJ;
    if (what == shifted_tile) b_col = b_col + T * RJ;
    if (what == unaligned_tile) a_row = a_row - 1;
    acc.cache_shared(A, k0, {T * RI + (what == unaligned_tile ? 1 : 0), kshape}, {a_row, k0 * KB}, true);
    acc.cache_shared(B, k0, {KB, T * RJ}, {k0 * KB, b_col});

    tiramisu::codegen({A.get_buffer(), B.get_buffer(), C.get_buffer()}, "build/" + name + ".o", true);
}

// D(i, j) = 2 * acc(i, 0): race-free as scheduled (a thread owns row i), but the value is not the
// one the epilogue of an MFMA tile has at hand for element (i, j).
static void generate_epilogue_other_element(const std::string &name)
{
    const int M = 128, N = 64, K = 32;
    tiramisu::init(name);
    var i("i", 0, M), j("j", 0, N), k("k", 0, K), i0("i0"), i1("i1");
    input A({i, k}, p_float32);
    input B({k, j}, p_float32);
    computation acc_init({i, j}, (float)0);
    computation acc({i, j, k}, p_float32);
    acc.store_in(acc_init.get_buffer(), {i, j});
    acc.set_expression(acc(i, j, 0) + A(i, k) * B(k, j));
    computation D({i, j}, acc(i, 0, 0) * expr((float)2));
    for (buffer *b : {A.get_buffer(), B.get_buffer(), acc_init.get_buffer(), D.get_buffer()}) b->tag_gpu_global();
    for (computation *c : {&acc_init, &acc, &D}) {
        c->split(i, 64, i0, i1);
        c->tag_gpu_level(i0, i1);
    }
    acc_init.then(acc, i1).then(D, i1);
    tiramisu::codegen({A.get_buffer(), B.get_buffer(), acc_init.get_buffer(), D.get_buffer()}, "build/" + name + ".o", true);
}

int main()
{
    generate_epilogue_other_element("proofs_epilogue_other_element");
    generate("proofs_sound", none);
    generate("proofs_short_tile", short_tile);
    generate("proofs_shifted_tile", shifted_tile);
    generate("proofs_unaligned_tile", unaligned_tile);
    generate("proofs_shared_register", shared_register);
    return 0;
}
