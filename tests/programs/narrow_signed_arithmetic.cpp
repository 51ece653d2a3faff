// Products of signed 8- and 16-bit values followed by an operation that depends on the sign of the truncated product:
//   half = (a * b) / 2, rem = (a * b) % 3, shifted = (a * b) >> 1, prod = a * b, square_half = (a * a) / 2
// for all 256 x 256 pairs of int8 values (a = i - 128, b = j - 128 come in as inputs) and, as int16, for a and b
// scaled by 211 and 173.  Tiramisu expressions keep their type: the product wraps to 8 (16) bits before it is
// divided (c_printer casts after every operation).  hipcc 7.2 for gfx950 computed (int8_t)((int8_t)(a * b) / 2) as
// x + 3 for most x when this test was written; the printer passes such products through an empty asm statement.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

template <primitive_t T>
static void generate(const std::string &name)
{
    const int N = 256;
    tiramisu::init(name);
    var i("i", 0, N), j("j", 0, N), i0("i0"), j0("j0"), i1("i1"), j1("j1");
    input A("A", {i, j}, T), B("B", {i, j}, T);
    computation half("half", {i, j}, (B(i, j) * A(i, j)) / cast(T, expr(2)));
    computation rem("rem", {i, j}, (B(i, j) * A(i, j)) % cast(T, expr(3)));
    computation shifted("shifted", {i, j}, (B(i, j) * A(i, j)) >> cast(T, expr(1)));
    computation prod("prod", {i, j}, B(i, j) * A(i, j));
    computation square_half("square_half", {i, j}, (A(i, j) * A(i, j)) / cast(T, expr(2)));
    std::vector<computation *> all = {&half, &rem, &shifted, &prod, &square_half};
    std::vector<buffer *> args = {A.get_buffer(), B.get_buffer()};
    for (computation *c : all) args.push_back(c->get_buffer());
#ifndef TIRAMISU_TARGET_CPU
    for (buffer *b : args) b->tag_gpu_global();
    for (computation *c : all) c->gpu_tile(i, j, 16, 16, i0, j0, i1, j1);
    half.then(rem, j1).then(shifted, j1).then(prod, j1).then(square_half, j1);
    tiramisu::codegen(args, "build/" + name + ".o", true);
#else
    half.then(rem, j).then(shifted, j).then(prod, j).then(square_half, j);
    tiramisu::codegen(args, "build/" + name + "_cpu.o", false);
#endif
}

int main(int argc, char **argv)
{
    tiramisu::backend_options_from_command_line(argc, argv);
    generate<p_int8>("narrow_products_int8");
    generate<p_int16>("narrow_products_int16");
    return 0;
}
