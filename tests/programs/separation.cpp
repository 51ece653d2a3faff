// separate / separateAndSplit / separate_at: a loop cut into a full part (whole groups of the split factor, counted
// from the loop's lower bound) and a remainder computed by a definition of its own (reference:
// tiramisu_core.cpp:746-870, :872-1010, :6103-6240), plus a duplicate restricted to a part of the domain.
// Every function computes out(i, j) = 100 * i + j over its domain, so a piece that is lost or computed over the
// wrong range shows in the result; the generator also writes, per function, which iterations of j each piece takes
// (build/separation.json), which the test compares with the definition.
// CPU_ONLY_PROGRAM: the pieces are a property of the shared front-end.
#include <tiramisu/tiramisu.h>

#include <cstdio>
#include <fstream>

using namespace tiramisu;

static std::ofstream report;
static bool first_entry = true;

// the ranges of j and i that each piece executes
static void describe(const std::string &fn, function *f) {
    report << (first_entry ? "" : ",\n") << "  \"" << fn << "\": [";
    first_entry = false;
    bool first_piece = true;
    for (auto c : f->get_computations()) {
        if (!c->should_schedule_this_computation() || c->get_name().find("out") == std::string::npos) continue;
        long lo = 0, hi = -1, row_lo = 0, row_hi = -1;
        c->executed_range(1, lo, hi);
        c->executed_range(0, row_lo, row_hi);
        report << (first_piece ? "" : ", ") << "{\"name\": \"" << c->get_name() << "\", \"levels\": " << c->get_loop_levels_number() << ", \"first\": " << lo
               << ", \"last\": " << hi << ", \"first_row\": " << row_lo << ", \"last_row\": " << row_hi << "}";
        first_piece = false;
    }
    report << "]";
}

int main()
{
    report.open("build/separation.json");
    report << "{\n";
    {   // 14 iterations by 4: full part [0, 12), remainder [12, 14)
        tiramisu::init("sep_split");
        var i("i", 0, 6), j("j", 0, 14), jo("jo"), ji("ji");
        computation out("out", {i, j}, cast(p_int32, i) * 100 + cast(p_int32, j));
        buffer b("b", {6, 14}, p_int32, a_output);
        out.store_in(&b);
        const bool happened = out.separateAndSplit(j, 4, jo, ji);
        if (!happened) return 1;
        out.tag_vector_level(ji, 4);
        describe("sep_split", global::get_implicit_function());
        tiramisu::codegen({&b}, "build/sep_split_cpu.o", false);
    }
    {   // a loop that starts at 3: groups are counted from 3, full part [3, 15), remainder [15, 17)
        tiramisu::init("sep_lower");
        var i("i", 0, 6), j("j", 3, 17), jo("jo"), ji("ji");
        computation out("out", {i, j}, cast(p_int32, i) * 100 + cast(p_int32, j));
        buffer b("b", {6, 17}, p_int32, a_output);
        out.store_in(&b);
        if (!out.separateAndSplit(j, 4, jo, ji)) return 1;
        describe("sep_lower", global::get_implicit_function());
        tiramisu::codegen({&b}, "build/sep_lower_cpu.o", false);
    }
    {   // a multiple of the factor: nothing to separate, only the split
        tiramisu::init("sep_exact");
        var i("i", 0, 6), j("j", 0, 16), jo("jo"), ji("ji");
        computation out("out", {i, j}, cast(p_int32, i) * 100 + cast(p_int32, j));
        buffer b("b", {6, 16}, p_int32, a_output);
        out.store_in(&b);
        if (!out.separateAndSplit(j, 4, jo, ji)) return 1;
        describe("sep_exact", global::get_implicit_function());
        tiramisu::codegen({&b}, "build/sep_exact_cpu.o", false);
    }
    {   // a loop not longer than the factor stays whole
        tiramisu::init("sep_short");
        var i("i", 0, 6), j("j", 0, 3), jo("jo"), ji("ji");
        computation out("out", {i, j}, cast(p_int32, i) * 100 + cast(p_int32, j));
        buffer b("b", {6, 3}, p_int32, a_output);
        out.store_in(&b);
        if (out.separateAndSplit(j, 4, jo, ji)) return 1;
        describe("sep_short", global::get_implicit_function());
        tiramisu::codegen({&b}, "build/sep_short_cpu.o", false);
    }
    {   // separate() alone, on the outer loop, with an explicit extent: [0, 4), [4, 6)
        tiramisu::init("sep_outer");
        var i("i", 0, 6), j("j", 0, 14);
        computation out("out", {i, j}, cast(p_int32, i) * 100 + cast(p_int32, j));
        buffer b("b", {6, 14}, p_int32, a_output);
        out.store_in(&b);
        out.separate(0, expr((int32_t)6), 4);
        out.get_update(1).interchange(i, j);        // the pieces are scheduled on their own
        describe("sep_outer", global::get_implicit_function());
        tiramisu::codegen({&b}, "build/sep_outer_cpu.o", false);
    }
    {   // three pieces at given points: [0, 4), [4, 9), [9, 14)
        tiramisu::init("sep_at");
        var i("i", 0, 6), j("j", 0, 14);
        computation out("out", {i, j}, cast(p_int32, i) * 100 + cast(p_int32, j));
        buffer b("b", {6, 14}, p_int32, a_output);
        out.store_in(&b);
        out.separate_at(j, {expr((int32_t)4), expr((int32_t)9)}, expr((int32_t)14));
        describe("sep_at", global::get_implicit_function());
        tiramisu::codegen({&b}, "build/sep_at_cpu.o", false);
    }
    {   // a duplicate over a part of the domain writes 1000 more there, after the original
        tiramisu::init("sep_duplicate");
        var i("i", 0, 6), j("j", 0, 14);
        computation out("out", {i, j}, cast(p_int32, i) * 100 + cast(p_int32, j));
        buffer b("b", {6, 14}, p_int32, a_output);
        out.store_in(&b);
        computation *copy = out.duplicate("{ out[i, j] : 2 <= i <= 3 and 5 <= j <= 7 }", "");
        if (copy != out.select(1)) return 1;
        copy->set_expression(cast(p_int32, i) * 100 + cast(p_int32, j) + 1000);
        copy->after(out, computation::root);
        describe("sep_duplicate", global::get_implicit_function());
        tiramisu::codegen({&b}, "build/sep_duplicate_cpu.o", false);
    }
    report << "\n}\n";
    report.close();
    return 0;
}
