// The dependence analysis and the legality checks built on it, asked about small programs whose answers can be
// read off the loops.  The program writes one "case=answer" line per question to build/dependence_checks.txt;
// run with the argument "refuse" (and TIRAMISU_HIP_CHECK_MAPPED_LOOPS set) it generates GPU code for a row scan
// whose thread loop carries a dependence, which codegen must refuse.
#include <tiramisu/tiramisu.h>

#include <fstream>

using namespace tiramisu;

static std::ofstream report;

static void say(const std::string &what, bool answer) { report << what << "=" << (answer ? "yes" : "no") << "\n"; }

// S(i,j) = S(i-1,j) + S(i,j-1), in place: distances (1,0) and (0,1)
static void wavefront()
{
    tiramisu::init("wavefront");
    var i("i", 1, 40), j("j", 1, 30), i1("i1"), j1("j1"), jr("jr");
    input A("A", {var("y", 0, 40), var("x", 0, 30)}, p_float32);
    computation S("S", {i, j}, A(i - 1, j) + A(i, j - 1));
    S.store_in(A.get_buffer());
    function *f = global::get_implicit_function();
    perform_full_dependency_analysis();
    prepare_schedules_for_legality_checks();
    say("wavefront.as_written.legal", check_legality_of_function());
    say("wavefront.as_written.i_parallel", loop_parallelization_is_legal(i, {&S}));
    say("wavefront.as_written.j_parallel", loop_parallelization_is_legal(j, {&S}));
    say("wavefront.as_written.j_unrollable", loop_unrolling_is_legal(j, {&S}));
    report << "wavefront.dependences:\n" << f->dependences_as_text();      // row 0 and column 0 come from outside
    S.interchange(i, j);                     // (1,0),(0,1) -> (0,1),(1,0)
    say("wavefront.interchanged.legal", check_legality_of_function());
    S.interchange(j, i);
    S.skew(i, j, 1, 1, i1, j1);              // i1 = i + j, j1 = j: distances (1,0) and (1,1)
    say("wavefront.skewed.legal", check_legality_of_function());
    say("wavefront.skewed.outer_parallel", loop_parallelization_is_legal(i1, {&S}));
    say("wavefront.skewed.inner_parallel", loop_parallelization_is_legal(j1, {&S}));
    say("wavefront.skewed.inner_unrollable", loop_unrolling_is_legal(j1, {&S}));
    say("wavefront.skewed.inner_vectorizable", loop_vectorization_is_legal(j1, {&S}));
}

// skewings found from the distances: (1,0),(0,1) need a > 0 and b > 0 to be carried by the outer loop; a diagonal
// recurrence with distance (1,1) only leaves the outer loop free after i - j
static void list(const std::string &what, const std::vector<std::pair<int, int>> &v)
{
    report << what << "=" << v.size();
    for (auto &p : v) report << " (" << p.first << "," << p.second << ")";
    report << "\n";
}

static void skewing()
{
    {
        tiramisu::init("skewing_wavefront");
        var i("i", 1, 40), j("j", 1, 30);
        input A("A", {var("y", 0, 40), var("x", 0, 30)}, p_float32);
        computation S("S", {i, j}, A(i - 1, j) + A(i, j - 1));
        S.store_in(A.get_buffer());
        perform_full_dependency_analysis();
        auto found = global::get_implicit_function()->skewing_local_solver({&S}, i, j, 2);
        list("skewing.wavefront.outer_parallel", std::get<0>(found));
        list("skewing.wavefront.inner_parallel", std::get<1>(found));
        list("skewing.wavefront.locality", std::get<2>(found));
        auto positive = global::get_implicit_function()->skewing_local_solver_positive({&S}, i, j, 1);
        report << "skewing.wavefront.positive.inner_parallel=" << std::get<1>(positive).size();
        for (auto &t : std::get<1>(positive)) report << " (" << std::get<0>(t) << "," << std::get<1>(t) << "," << std::get<2>(t) << "," << std::get<3>(t) << ")";
        report << "\n";
    }
    {
        tiramisu::init("skewing_diagonal");
        var i("i", 1, 40), j("j", 1, 30), i1("i1"), j1("j1");
        input A("A", {var("y", 0, 40), var("x", 0, 30)}, p_float32);
        computation S("S", {i, j}, A(i - 1, j - 1) * 2.0f);
        S.store_in(A.get_buffer());
        perform_full_dependency_analysis();
        auto found = global::get_implicit_function()->skewing_local_solver({&S}, i, j, 1);
        list("skewing.diagonal.outer_parallel", std::get<0>(found));
        if (!std::get<0>(found).empty()) {
            S.skew(i, j, std::get<0>(found)[0].first, std::get<0>(found)[0].second, i1, j1);
            prepare_schedules_for_legality_checks();
            say("skewing.diagonal.skewed.legal", check_legality_of_function());
            say("skewing.diagonal.skewed.outer_parallel", loop_parallelization_is_legal(i1, {&S}));
        }
    }
    {
        tiramisu::init("skewing_nothing_to_do");
        var i("i", 1, 40), j("j", 1, 30);
        input A("A", {var("y", 0, 41), var("x", 0, 31)}, p_float32);
        computation B("B", {i, j}, A(i - 1, j) + A(i + 1, j + 1));
        perform_full_dependency_analysis();
        auto found = global::get_implicit_function()->skewing_local_solver({&B}, i, j, 2);
        report << "skewing.out_of_place.total=" << std::get<0>(found).size() + std::get<1>(found).size() + std::get<2>(found).size() << "\n";
    }
}

// the schedule of the reference's tests/test_133.cpp (134-140 vary it): the recurrence above, skew(i, j, 1) -- which
// keeps i outermost, (1,0),(0,1) -> (1,1),(0,1) -- and the outer loop tagged parallel although it carries (1,1)
static void skewed_outer_loop_tagged_parallel()
{
    tiramisu::init("skewed_outer_parallel");
    var i("i", 1, 40), j("j", 1, 40), ni("ni"), nj("nj");
    input A("A", {var("y", 0, 40), var("x", 0, 40)}, p_uint8);
    computation S("S", {i, j}, A(i - 1, j) + A(i, j - 1));
    S.store_in(A.get_buffer());
    perform_full_dependency_analysis();
    S.skew(i, j, 1, ni, nj);
    prepare_schedules_for_legality_checks();
    say("test_133.order_legal", check_legality_of_function());
    say("test_133.ni_parallel", loop_parallelization_is_legal(ni, {&S}));
    say("test_133.nj_parallel", loop_parallelization_is_legal(nj, {&S}));
}

// the same recurrence with the inner loop run backwards: (0,1) becomes (0,-1)
static void reversed()
{
    tiramisu::init("reversed");
    var i("i", 1, 40), j("j", 1, 30), jr("jr");
    input A("A", {var("y", 0, 40), var("x", 0, 30)}, p_float32);
    computation S("S", {i, j}, A(i - 1, j) + A(i, j - 1));
    S.store_in(A.get_buffer());
    perform_full_dependency_analysis();
    S.loop_reversal(j, jr);
    prepare_schedules_for_legality_checks();
    say("reversed.legal", check_legality_of_function());
}

// out of place: nothing read is ever written
static void out_of_place()
{
    tiramisu::init("out_of_place");
    var i("i", 1, 39), j("j", 1, 29), i0("i0"), j0("j0"), i1("i1"), j1("j1");
    input A("A", {var("y", 0, 40), var("x", 0, 30)}, p_float32);
    computation B("B", {i, j}, A(i - 1, j) + A(i + 1, j) + A(i, j - 1) + A(i, j + 1));
    function *f = global::get_implicit_function();
    perform_full_dependency_analysis();
    B.tile(i, j, 8, 8, i0, j0, i1, j1);
    prepare_schedules_for_legality_checks();
    say("out_of_place.tiled.legal", check_legality_of_function());
    say("out_of_place.tiled.i0_parallel", loop_parallelization_is_legal(i0, {&B}));
    say("out_of_place.tiled.j1_parallel", loop_parallelization_is_legal(j1, {&B}));
    report << "out_of_place.dependences:\n" << f->dependences_as_text();
}

// P(i) = A(i), Q(i) = P(i + 2): fused in one loop Q runs two iterations early; a shift by 2 repairs it
static void fusion()
{
    tiramisu::init("fusion");
    var i("i", 0, 50), i_all("i", 0, 60);
    input A("A", {var("x", 0, 60)}, p_float32);
    computation P("P", {i_all}, A(i_all) * 2.0f);
    computation Q("Q", {i}, P(i + 2) + 1.0f);
    P.then(Q, computation::root);
    function *f = global::get_implicit_function();
    perform_full_dependency_analysis();
    prepare_schedules_for_legality_checks();
    say("fusion.one_after_the_other.legal", check_legality_of_function());
    P.then(Q, i);
    prepare_schedules_for_legality_checks(true);
    say("fusion.fused.legal", f->check_partial_legality_in_function({&P, &Q}));
    say("fusion.fused.P_to_Q_legal", P.involved_subset_of_dependencies_is_legal(&Q));
    auto shifts = f->correcting_loop_fusion_with_shifting({&P}, Q, {i});
    report << "fusion.shifts=" << shifts.size();
    for (auto &s : shifts) report << " " << std::get<0>(s).get_name() << ":" << std::get<1>(s);
    report << "\n";
    for (auto &s : shifts) Q.shift(std::get<0>(s), std::get<1>(s));
    say("fusion.shifted.legal", check_legality_of_function());
}

// ---- loops mapped to the GPU
static void scan_rows(bool generate)
{
    tiramisu::init("scan_rows");
    var i("i", 0, 64), j("j", 1, 64);
    input A("A", {var("y", 0, 64), var("x", 0, 64)}, p_float32);
    computation S("S", {i, j}, A(i, j) + A(i, j - 1));     // reads what the iteration before wrote
    S.store_in(A.get_buffer());
    A.get_buffer()->tag_gpu_global();
    S.tag_gpu_level(i, j);
    if (generate) {
        tiramisu::codegen({A.get_buffer()}, "build/scan_rows_refused.o", true);
        return;
    }
    function *f = global::get_implicit_function();
    f->gen_ordering_schedules();
    for (auto &line : f->gpu_mapped_loops_that_carry_dependences()) report << "mapped.scan_rows: " << line << "\n";
}

static void mapped_loops()
{
    scan_rows(false);
    function *f;

    tiramisu::init("row_sums_mapped");
    var i("i", 0, 64), j("j", 0, 64);
    input B("B", {i, j}, p_float32);
    computation s_init("s_init", {i}, expr((float)0));
    computation s("s", {i, j}, p_float32);
    s.store_in(s_init.get_buffer(), {i});
    s.set_expression(s(i, 0) + B(i, j));
    s_init.then(s, computation::root);
    s.tag_gpu_level(i, j);
    f = global::get_implicit_function();
    f->gen_ordering_schedules();
    for (auto &line : f->gpu_mapped_loops_that_carry_dependences()) report << "mapped.row_sums: " << line << "\n";

    // a permutation in place through an index table: the element an iteration reads may be one that another writes
    tiramisu::init("gather_in_place");
    var k("k", 0, 64), k0("k0"), k1("k1");
    input T("T", {k}, p_int32);
    input V("V", {k}, p_float32);
    computation G("G", {k}, V(T(k)) + 1.0f);
    G.store_in(V.get_buffer());
    G.split(k, 16, k0, k1);
    G.tag_gpu_level(k0, k1);
    f = global::get_implicit_function();
    f->gen_ordering_schedules();
    for (auto &line : f->gpu_mapped_loops_that_carry_dependences()) report << "mapped.gather: " << line << "\n";

    tiramisu::init("scale_mapped");
    input C("C", {i, j}, p_float32);
    computation D("D", {i, j}, C(i, j) * 3.0f);
    D.tag_gpu_level(i, j);
    f = global::get_implicit_function();
    f->gen_ordering_schedules();
    report << "mapped.scale.findings=" << f->gpu_mapped_loops_that_carry_dependences().size() << "\n";
}

int main(int argc, char **argv)
{
    if (argc > 1 && std::string(argv[1]) == "refuse") {
        scan_rows(true);
        return 0;
    }
    report.open("build/dependence_checks.txt");
    wavefront();
    reversed();
    out_of_place();
    fusion();
    skewed_outer_loop_tagged_parallel();
    skewing();
    mapped_loops();
    report.close();
    return 0;
}
