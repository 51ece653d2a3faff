// compute_at with redundant computation (reference: tiramisu_core.cpp:5262-5660): a two-stage blur whose first
// stage is computed inside the loop nest of the second.  What the consumer's iterations of the chosen level read
// that the producer does not compute in the same iteration is computed by a duplicate, shifted into an earlier or
// the same iteration; the programs differ in the level and in what lies outside.
// CPU_ONLY_PROGRAM: the duplicate and its schedule are a property of the shared front-end.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

static const int H = 20, W = 24;

struct blur {
    var y, x, yi, xi;
    buffer b_in, b_bx, b_by;
    input in;
    computation bx, by;
    blur()
        : y("y", 0, H), x("x", 0, W), yi("yi", 0, H + 2), xi("xi", 0, W + 2),
          b_in("b_in", {H + 2, W + 2}, p_int32, a_input), b_bx("b_bx", {H + 2, W}, p_int32, a_output),
          b_by("b_by", {H, W}, p_int32, a_output), in("in", {yi, xi}, p_int32),
          bx("bx", {yi, x}, in(yi, x) + in(yi, x + 1) + in(yi, x + 2)),
          by("by", {y, x}, bx(y, x) + bx(y + 1, x) + bx(y + 2, x))
    {
        in.store_in(&b_in);
        bx.store_in(&b_bx);
        by.store_in(&b_by);
    }
    void finish(const std::string &fn) { tiramisu::codegen({&b_in, &b_bx, &b_by}, "build/" + fn + "_cpu.o", false); }
};

int main()
{
    {   // per row: row y of by needs rows y, y + 1, y + 2 of bx; the duplicate computes a row two iterations early
        tiramisu::init("compute_at_row");
        blur p;
        p.bx.compute_at(p.by, p.y);
        p.finish("compute_at_row");
    }
    {   // per row of 8x8 tiles: the two rows below a tile come from the duplicate
        tiramisu::init("compute_at_tile");
        blur p;
        var y0("y0"), x0("x0"), y1("y1"), x1("x1");
        p.bx.tile(p.yi, p.x, 8, 8, y0, x0, y1, x1);
        p.by.tile(p.y, p.x, 8, 8, y0, x0, y1, x1);
        p.bx.compute_at(p.by, x0);
        p.finish("compute_at_tile");
    }
    {   // nothing missing (the consumer reads what the same iteration produces): ordering only
        tiramisu::init("compute_at_same");
        var y("y", 0, H), x("x", 0, W);
        input in("in", {y, x}, p_int32);
        computation a("a", {y, x}, in(y, x) * 2), c("c", {y, x}, a(y, x) + 1);
        buffer b_in("b_in", {H, W}, p_int32, a_input), b_a("b_a", {H, W}, p_int32, a_output), b_c("b_c", {H, W}, p_int32, a_output);
        in.store_in(&b_in);
        a.store_in(&b_a);
        c.store_in(&b_c);
        a.compute_at(c, x);
        if (a.select(0) != &a) return 1;
        tiramisu::codegen({&b_in, &b_a, &b_c}, "build/compute_at_same_cpu.o", false);
    }
    {   // storage_fold: rows of bx kept modulo 4 while by follows three rows behind in the same row loop
        tiramisu::init("storage_fold_rows");
        blur p;
        p.bx.compute_at(p.by, p.y);
        p.bx.storage_fold(p.yi, 4);
        p.finish("storage_fold_rows");
    }
    return 0;
}
