// Pattern-directed kernel emitters.  A GPU-mapped loop nest is handed to these before the
// schedule-faithful emitter; each one checks -- on the computations' expressions, iteration
// domains and store relations, with isl where sets and maps are compared -- that the nest is of
// its kind, and only then replaces it by kernels shaped for gfx950.  Anything that fails a check
// falls back to the generic emitter, which reproduces the reference's behaviour.
#include <dlfcn.h>
#include <unistd.h>
#include <algorithm>
#include <cstdlib>
#include <sstream>

#include "hip_backend.h"
#include "stencil_plan.h"
#include <tiramisu/isl_api.h>
#include "kernels/target_gfx950.h"
#include "util.h"

namespace tiramisu {
namespace hipgen {

using lir::leaf_kind;
using lir::node;
using lir::node_kind;
using lir::node_ptr;

#ifndef TIRAMISU_AMD_KERNEL_DIR
#define TIRAMISU_AMD_KERNEL_DIR "."
#endif

#ifndef TIRAMISU_AMD_INCLUDE_DIR
#define TIRAMISU_AMD_INCLUDE_DIR "."
#endif

// A directory of files that generated code needs at code-generation time.  An installed library (lib/libtiramisu.so
// with share/ and include/ beside lib/) finds them relative to its own file, so that an installation can be moved;
// a library in its build tree falls back to the source directories it was built from.
static std::string beside_library(const char *relative, const char *probe) {
    Dl_info info;
    if (!dladdr((void *)&beside_library, &info) || !info.dli_fname) return "";
    const std::string lib = info.dli_fname;
    const size_t slash = lib.rfind('/');
    const std::string dir = (slash == std::string::npos ? std::string(".") : lib.substr(0, slash)) + "/" + relative;
    if (access((dir + "/" + probe).c_str(), R_OK) != 0) return "";
    char *real = realpath(dir.c_str(), nullptr);
    const std::string out = real ? real : dir;
    free(real);
    return out;
}

// the kernel headers (generated device code includes them by file name; the device compiler gets this directory as -I)
std::string kernel_dir() {
    if (const char *e = std::getenv("TIRAMISU_AMD_KERNEL_DIR")) return e;
    const std::string installed = beside_library("../share/tiramisu/kernels", "gemm_mfma.hip.h");
    return installed.empty() ? TIRAMISU_AMD_KERNEL_DIR : installed;
}

// tiramisu_hip_wrappers.h for the generated host code
std::string include_dir() {
    if (const char *e = std::getenv("TIRAMISU_AMD_INCLUDE")) return e;
    const std::string installed = beside_library("../include", "tiramisu_hip_wrappers.h");
    return installed.empty() ? TIRAMISU_AMD_INCLUDE_DIR : installed;
}

void add_include_once(context &ctx, const std::string &line) {
    if (ctx.include_once.insert(line).second) ctx.includes += line + "\n";
}

namespace {


int env_int(const char *name, int dflt) {
    const char *e = backend_option(name);
    return e ? std::atoi(e) : dflt;
}

// e == v + c ?
bool var_plus_const(const expr &e_in, const std::string &v, long &c) {
    expr e = lir::simplify(e_in);
    if (e.get_expr_type() == e_var && e.get_name() == v) { c = 0; return true; }
    if (e.get_expr_type() != e_op) return false;
    if (e.get_op_type() == o_add || e.get_op_type() == o_sub) {
        const expr &a = e.get_operand(0), &b = e.get_operand(1);
        long sign = e.get_op_type() == o_add ? 1 : -1;
        if (a.get_expr_type() == e_var && a.get_name() == v && b.is_integer_literal()) { c = sign * b.get_int_val(); return true; }
        if (sign == 1 && b.get_expr_type() == e_var && b.get_name() == v && a.is_integer_literal()) { c = a.get_int_val(); return true; }
    }
    return false;
}

bool literal_box(computation *C, std::vector<long> &lo, std::vector<long> &hi) {
    isl_set *d = C->get_iteration_domain();
    int n = isl_set_dim(d, isl_dim_set);
    std::ostringstream box;
    box << "{ " << C->get_name() << "[";
    for (int i = 0; i < n; i++) box << (i ? "," : "") << "d" << i;
    box << "] : ";
    for (int i = 0; i < n; i++) {
        isl_val *mn = isl_set_dim_min_val(isl_set_copy(d), i);
        isl_val *mx = isl_set_dim_max_val(isl_set_copy(d), i);
        bool ok = mn && mx && isl_val_is_int(mn) == isl_bool_true && isl_val_is_int(mx) == isl_bool_true;
        if (ok) { lo.push_back(isl_val_get_num_si(mn)); hi.push_back(isl_val_get_num_si(mx)); }
        isl_val_free(mn);
        isl_val_free(mx);
        if (!ok) return false;
        box << (i ? " and " : "") << lo[i] << " <= d" << i << " <= " << hi[i];
    }
    box << " }";
    isl_set *b = isl_set_read_from_str(C->get_ctx(), box.str().c_str());
    bool eq = b && isl_set_is_equal(d, b) == isl_bool_true;
    isl_set_free(b);
    return eq;
}

bool access_equals(computation *C, const std::string &expected) {
    isl_map *m = isl_map_read_from_str(C->get_ctx(), expected.c_str());
    if (!m) return false;
    bool eq = isl_map_is_equal(m, C->get_access_relation()) == isl_bool_true;
    isl_map_free(m);
    return eq;
}

// Dataflow check of the time-iterated stencil, on the program as scheduled: with S stored at B[t mod 2, y, x] and
// reading B[(t-1) mod 2, y+dy, x+dx], the last write that each read sees (isl's flow analysis over S's
// schedule) must be exactly the previous step's instance at the offset cell, wherever that cell is in the
// iteration domain -- i.e. the flow dependences are { S[t-1, y+dy, x+dx] -> S[t, y, x] } and nothing else.
// Cells outside the domain have no source: they hold what the buffer held on entry.
bool flow_is_previous_step(computation *S, buffer *B, const std::vector<std::pair<long, long>> &taps) {
    isl_ctx *ctx = S->get_ctx();
    const std::string s = S->get_name(), b = B->get_name();
    auto restricted = [&](const std::string &text) {
        isl_union_map *m = isl_union_map_read_from_str(ctx, text.c_str());
        return m ? isl_union_map_intersect_domain(m, isl_union_set_from_set(isl_set_copy(S->get_iteration_domain()))) : nullptr;
    };
    isl_union_map *writes = restricted("{ " + s + "[t,y,x] -> " + b + "[t mod 2, y, x] }");
    isl_union_map *reads = nullptr, *expected = nullptr;
    for (auto &tap : taps) {
        const std::string dy = std::to_string(tap.first), dx = std::to_string(tap.second);
        isl_union_map *r = restricted("{ " + s + "[t,y,x] -> " + b + "[(t - 1) mod 2, y + (" + dy + "), x + (" + dx + ")] }");
        // source instance -> sink instance, both inside the domain
        isl_union_map *e = restricted("{ " + s + "[t,y,x] -> " + s + "[t + 1, y - (" + dy + "), x - (" + dx + ")] }");
        if (e) e = isl_union_map_intersect_domain(isl_union_map_reverse(e), isl_union_set_from_set(isl_set_copy(S->get_iteration_domain())));
        if (e) e = isl_union_map_reverse(e);
        reads = reads ? isl_union_map_union(reads, r) : r;
        expected = expected ? isl_union_map_union(expected, e) : e;
    }
    isl_map *sched = isl_map_project_out(isl_map_copy(S->get_schedule()), isl_dim_out, 0, 1);   // the duplicate dimension
    sched = isl_map_intersect_domain(sched, isl_set_copy(S->get_iteration_domain()));
    bool ok = false;
    if (writes && reads && expected && sched) {
        isl_union_access_info *info = isl_union_access_info_from_sink(reads);
        info = isl_union_access_info_set_must_source(info, writes);
        info = isl_union_access_info_set_schedule_map(info, isl_union_map_from_map(sched));
        reads = writes = nullptr;
        sched = nullptr;
        isl_union_flow *flow = isl_union_access_info_compute_flow(info);
        if (flow) {
            isl_union_map *dep = isl_union_flow_get_must_dependence(flow);
            ok = dep && isl_union_map_is_equal(dep, expected) == isl_bool_true;
            if (dep) isl_union_map_free(dep);
            isl_union_flow_free(flow);
        }
    }
    if (writes) isl_union_map_free(writes);
    if (reads) isl_union_map_free(reads);
    if (expected) isl_union_map_free(expected);
    if (sched) isl_map_free(sched);
    return ok;
}

void leaves_under(const node_ptr &n, std::vector<node_ptr> &out, bool &has_cond) {
    lir::walk(n, [&](const node_ptr &x) {
        if (x->kind == node_kind::leaf) out.push_back(x);
        if (x->kind == node_kind::cond) has_cond = true;
    });
}

}  // namespace

// ------------------------------------------------------------------------------------------
// Stencil over a ping-pong pair of planes inside a host time loop:
//     S(t, y, x) = f( S(t-1, y+dy, x+dx) ... ),   S stored at B[t mod 2, y, x].
// Every read at step t is of step t-1 within a constant radius, so all flow dependences have
// distance (1, dy, dx) (flow_is_previous_step checks that on the scheduled program with isl's dataflow
// analysis) and overlapped time tiles are legal; the time loop is replaced by
// launches that each advance several steps (see kernels/stencil2d_regs.hip.h).  The second form is a single
// step out of place:  S(y, x) = f( I(y+dy, x+dx) ... )  with I and S in buffers of their own.
bool emit_stencil(context &ctx, const node_ptr &root, const node_ptr &time_loop, launch_plan &plan) {
    // either a host time loop around a mapped nest, or a mapped nest whose time step is fixed
    // (a one-step time loop has no loop node in the AST)
    if ((!time_loop && !root) || (time_loop && root)) return false;
    if (backend_option("TIRAMISU_NO_STENCIL")) return false;
    function *f = ctx.f;
    const node_ptr scope = time_loop ? time_loop->body : root;
    std::vector<node_ptr> leaves;
    bool has_cond = false;
    leaves_under(scope, leaves, has_cond);
    if (leaves.size() != 1 || has_cond) return false;
    node_ptr leaf = leaves[0];
    if (leaf->lkind != leaf_kind::assign || leaf->predicate.is_defined() || !leaf->lets.empty()) return false;
    // the nest below the time loop must be mapped to the GPU
    bool mapped = false;
    lir::walk(scope, [&](const node_ptr &x) { if (x->kind == node_kind::loop && x->gpu_block >= 0) mapped = true; });
    if (!mapped) return false;

    computation *S = leaf->comp;
    const auto &its = S->get_iteration_domain_dimension_names();
    // two forms: S(t, y, x) from S(t-1, ...) on a ping-pong pair of planes, and -- a single step out of place --
    // S(y, x) from another computation I(y+dy, x+dx) that lives in a buffer of its own
    const bool planar = its.size() == 2 && !time_loop;
    if ((its.size() != 3 && !planar) || S->get_data_type() != p_float32) return false;
    if (planar && backend_option("TIRAMISU_NO_SINGLE_STEP_STENCIL")) return false;
    if (!planar) {
        auto t_it = leaf->iterators.find(its[0]);
        if (t_it == leaf->iterators.end()) return false;
        if (time_loop) {
            if (t_it->second.get_expr_type() != e_var || t_it->second.get_name() != time_loop->iterator) return false;
        } else if (!lir::simplify(t_it->second).is_integer_literal()) {
            return false;
        }
    }
    const std::string &yi = its[planar ? 0 : 1], &xi = its[planar ? 1 : 2];

    // expression: reads of S at (t-1, y+dy, x+dx) -- of one other computation at (y+dy, x+dx) -- and float literals only
    int radius = 0;
    bool ok = true;
    std::string source_name = planar ? std::string() : S->get_name();
    std::vector<std::pair<long, long>> taps;
    std::function<expr(const expr &)> rewrite = [&](const expr &e) -> expr {
        if (!e.is_defined()) { ok = false; return e; }
        switch (e.get_expr_type()) {
        case e_val: return e;
        case e_op: {
            if (e.get_op_type() == o_access) {
                long dt = -1, dy, dx;
                if (planar && source_name.empty() && e.get_name() != S->get_name()) source_name = e.get_name();
                const size_t first = planar ? 0 : 1;
                if (e.get_name() != source_name || e.get_access().size() != its.size() || (!planar && !var_plus_const(e.get_access()[0], its[0], dt)) ||
                    !var_plus_const(e.get_access()[first], yi, dy) || !var_plus_const(e.get_access()[first + 1], xi, dx) || dt != -1) {
                    ok = false;
                    return e;
                }
                radius = std::max<long>(radius, std::max(std::labs(dy), std::labs(dx)));
                if (std::find(taps.begin(), taps.end(), std::make_pair(dy, dx)) == taps.end()) taps.push_back({dy, dx});
                return expr(o_call, "ST_AT", {expr((int32_t)dy), expr((int32_t)dx)}, p_float32);
            }
            if (e.get_op_type() == o_call) { ok = false; return e; }
            std::vector<expr> ops;
            for (auto &o : e.get_operands()) ops.push_back(rewrite(o));
            switch (ops.size()) {
            case 1: return e.get_op_type() == o_cast ? expr(o_cast, e.get_data_type(), ops[0]) : expr(e.get_op_type(), ops[0]);
            case 2: return expr(e.get_op_type(), ops[0], ops[1]).copy_with_type(e.get_data_type());
            case 3: return expr(e.get_op_type(), ops[0], ops[1], ops[2]);
            default: ok = false; return e;
            }
        }
        default: ok = false; return e;
        }
    };
    expr point = rewrite(S->get_expr());
    // radius 0 (a point-wise map of one buffer into another) is taken as a single step out of place only
    if (!ok || radius > 4 || (radius < 1 && !planar)) return false;

    // store relation and buffer
    buffer *B = leaf->lhs, *BI = nullptr;
    if (!B || B->get_location() != memory_location::global || B->get_n_dims() != (planar ? 2 : 3) || !B->has_constant_extents()) return false;
    if (!planar && lir::simplify(B->get_dim_sizes()[0]).get_int_val() != 2) return false;
    const long NY = lir::simplify(B->get_dim_sizes()[planar ? 0 : 1]).get_int_val(), NX = lir::simplify(B->get_dim_sizes()[planar ? 1 : 2]).get_int_val();
    if (planar) {
        // both computations stored as they are indexed, in two float buffers of the same shape
        if (source_name.empty()) return false;
        auto sources = f->get_computation_by_name(source_name);
        if (sources.size() != 1 || sources[0]->get_data_type() != p_float32) return false;
        BI = sources[0]->get_buffer();
        if (!BI || BI == B || BI->get_location() != memory_location::global || BI->get_n_dims() != 2 || !BI->has_constant_extents() ||
            BI->get_elements_type() != p_float32 || B->get_elements_type() != p_float32) return false;
        if (lir::simplify(BI->get_dim_sizes()[0]).get_int_val() != NY || lir::simplify(BI->get_dim_sizes()[1]).get_int_val() != NX) return false;
        if (!access_equals(S, "{ " + S->get_name() + "[y,x] -> " + B->get_name() + "[y, x] }") ||
            !access_equals(sources[0], "{ " + source_name + "[y,x] -> " + BI->get_name() + "[y, x] }")) return false;
    } else if (!access_equals(S, "{ " + S->get_name() + "[t,y,x] -> " + B->get_name() + "[t mod 2, y, x] }")) {
        return false;
    } else if (!backend_option("TIRAMISU_STENCIL_NO_FLOW_CHECK") && !flow_is_previous_step(S, B, taps)) {
        return false;
    }

    // iteration domain: a box that keeps the stencil inside the plane
    std::vector<long> lo, hi;
    if (!literal_box(S, lo, hi)) return false;
    if (planar) {                      // as one time step
        lo.insert(lo.begin(), 1);
        hi.insert(hi.begin(), 1);
    }
    if (lo[1] - radius < 0 || hi[1] + radius > NY - 1 || lo[2] - radius < 0 || hi[2] + radius > NX - 1) return false;

    // ---- plan.  On return both planes must hold exactly what the un-tiled loop leaves there: the last step in
    // one, the last but one in the other.  A launch between the two planes advances an odd number of steps.
    //  * With a third plane (allocated once per host thread, kept): odd chunks between the planes, the last of
    //    them into the third plane, and a final launch that reads the third plane and writes both planes (the
    //    values of its last step but one and of its last step), so no launch is spent on a single step.
    //  * Without (fewer than 3 steps, or TIRAMISU_STENCIL_TEMP_PLANE=0): odd chunks for all steps but the last,
    //    then the last step alone.
    const long T0 = lo[0], T1 = hi[0];
    const long steps = T1 - T0 + 1;
    // region staged by one workgroup: WAVES*ROWS rows by 256 columns (kernels/stencil2d_regs.hip.h)
    // fused launches: 8 wavefronts x 11 rows (a sweep over both put the optimum there); a single step out of place
    // streams, and 4 rows per thread keep more workgroups and loads in flight
    const int WAVES = env_int("TIRAMISU_STENCIL_WAVES", 8), ROWS = env_int("TIRAMISU_STENCIL_ROWS", planar ? 4 : 11);
    if (WAVES < 1 || WAVES > 16 || ROWS < radius || ROWS > 32) return false;
    const int LH = WAVES * ROWS, LW = 256;
    // most steps of one launch; a launch between the two planes takes the largest odd number below.  12: the final
    // launch writes two planes and has HBM time to cover one step more than the 11 of the others
    const int rcap = tstencil::step_cap(env_int("TIRAMISU_STENCIL_STEPS", 12), radius, LH);
    if (2 * radius >= LH) return false;
    typedef tstencil::chunk chunk;   // first step, number of steps, kernel mode (stencil2d_regs.hip.h)
    const bool temp_plane = !planar && steps >= 3 && rcap >= 2 && env_int("TIRAMISU_STENCIL_TEMP_PLANE", 1) != 0;
    const std::vector<chunk> chunks = tstencil::plan_time_loop(T0, steps, rcap, planar, temp_plane);

    c_printer dev;
    dev.fct = f;
    dev.device = true;
    const std::string point_text = dev.print(point);
    std::map<std::pair<int, int>, std::pair<kernel, kernel>> by_steps;   // (steps, mode) -> (interior tiles, tiles on the fixed boundary)
    std::ostringstream host;
    // one launch per chunk: the boundary slices ride behind the interior tiles (TIRAMISU_STENCIL_MERGE=0: two launches)
    const bool merge = env_int("TIRAMISU_STENCIL_MERGE", 1) != 0;
    static const char *const mode_text[] = {"", ", into a third plane", ", from a third plane into both planes", ", out of place"};
    host << "    {\n";
    if (temp_plane)
        host << "        static const char _st_site = 0;   // third plane: the runtime keeps it from call to call (per thread and stream)\n"
             << "        float *_st_temp = (float *)tiramisu_hip_kept_scratch(&_st_site, (uint64_t)" << NY << " * " << NX << " * sizeof(float), nullptr);\n";
    else if (!planar)
        host << "        float *_st_temp = nullptr;\n";
    for (auto &ch : chunks) {
        const std::pair<int, int> key(ch.steps, ch.mode);
        if (!by_steps.count(key)) {
            kernel k, ke;
            k.name = "_kernel_" + std::to_string(ctx.next_kernel_id());
            ke.name = "_kernel_" + std::to_string(ctx.next_kernel_id());
            const tstencil::launch_geometry g = tstencil::plan_launch(NY, NX, lo[1], hi[1], lo[2], hi[2], radius, ch.steps, WAVES, ROWS);
            const int TH = g.tile_rows, TW = g.tile_columns, rows_edge = g.rows_edge, TH_edge = g.slice_rows, edge_sub = g.slices;
            const long GX = g.tiles_x, GY = g.tiles_y, bx0 = g.ibx0, bx1 = g.ibx1, by0 = g.iby0, by1 = g.iby1;
            const long interior = g.interior, edge_tiles = g.edge_tiles;
            k.how = "stencil: " + std::to_string(ch.steps) + " time step(s) per launch, radius " + std::to_string(radius) +
                    ", tile " + std::to_string(TH) + "x" + std::to_string(TW) + " in registers, " + std::to_string(WAVES) +
                    " wavefronts x " + std::to_string(ROWS) + " rows, " + std::to_string(interior) + " interior tiles" + mode_text[ch.mode];
            ke.how = "stencil: the " + std::to_string(edge_tiles) + " tiles of " + k.name + "'s launch that touch the fixed boundary, in " +
                     std::to_string(edge_sub) + " slice(s) of " + std::to_string(TH_edge) + " rows each" +
                     (merge ? " (carried by " + k.name + "'s launch, after its interior tiles)" : "");
            std::ostringstream s;
            s << "#define ST_NAME " << k.name << "\n#define ST_NAME_EDGE " << ke.name << "\n#define ST_NY " << NY << "\n#define ST_NX " << NX
              << "\n#define ST_Y0 " << lo[1] << "\n#define ST_Y1 " << hi[1] << "\n#define ST_X0 " << lo[2] << "\n#define ST_X1 " << hi[2]
              << "\n#define ST_GX " << GX << "\n#define ST_GY " << GY << "\n#define ST_IBX0 " << bx0 << "\n#define ST_IBX1 " << bx1
              << "\n#define ST_IBY0 " << by0 << "\n#define ST_IBY1 " << by1 << "\n#define ST_W " << WAVES
              << "\n#define ST_MERGE " << (merge ? 1 : 0) << "\n#define ST_XCD " << env_int("TIRAMISU_STENCIL_XCD", 1) << "\n#define ST_OCC " << env_int("TIRAMISU_STENCIL_OCCUPANCY", 0) << "\n#define ST_STREAM " << env_int("TIRAMISU_STENCIL_STREAM", 2)
              << "\n#define ST_RPT " << ROWS << "\n#define ST_RPT_EDGE " << rows_edge << "\n#define ST_R " << ch.steps << "\n#define ST_MODE " << ch.mode << "\n#define ST_RAD " << radius
              << "\n#define ST_EXPR " << point_text << "\n#include \"stencil2d_regs.hip.h\"\n"
              << "#undef ST_NAME\n#undef ST_NAME_EDGE\n#undef ST_NY\n#undef ST_NX\n#undef ST_Y0\n#undef ST_Y1\n#undef ST_X0\n#undef ST_X1\n"
              << "#undef ST_GX\n#undef ST_GY\n#undef ST_IBX0\n#undef ST_IBX1\n#undef ST_IBY0\n#undef ST_IBY1\n#undef ST_W\n#undef ST_OCC\n#undef ST_STREAM\n"
              << "#undef ST_MERGE\n#undef ST_XCD\n#undef ST_RPT\n#undef ST_RPT_EDGE\n#undef ST_R\n#undef ST_MODE\n#undef ST_RAD\n#undef ST_EXPR\n";
            k.source = s.str();            // both kernels come from the one inclusion
            ke.source = "";
            for (kernel *q : {&k, &ke}) {
                // the kernel reads plane _st_src of its first buffer; out of place the source is that buffer and the
                // destination comes in the place of the third plane
                if (planar) q->params = {{true, BI->get_name(), p_float32}, {false, "_st_src", p_int32}, {true, B->get_name(), p_float32}};
                else q->params = {{true, B->get_name(), B->get_elements_type()}, {false, "_st_src", p_int32}, {true, "_st_temp", p_float32}};
                q->block[0] = std::to_string(64 * WAVES);
            }
            k.grid[0] = std::to_string(merge ? interior + edge_tiles * edge_sub : interior);
            ke.grid[0] = std::to_string(merge ? 0 : edge_tiles * edge_sub);
            by_steps[key] = {k, ke};
        }
        const long src = planar ? 0 : (((ch.first - 1) % 2) + 2) % 2;
        auto &pr = by_steps[key];
        host << "        {\n            const int32_t _st_src = " << src << ";  // steps " << ch.first << ".." << ch.first + ch.steps - 1 << "\n";
        if (pr.first.grid[0] != "0") host << launch_text(pr.first, "            ");
        if (pr.second.grid[0] != "0") host << launch_text(pr.second, "            ");
        host << "        }\n";
    }
    host << "    }\n";
    for (auto &kv : by_steps) { plan.kernels.push_back(kv.second.first); plan.kernels.push_back(kv.second.second); }
    plan.host_code = host.str();
    return true;
}

// ------------------------------------------------------------------------------------------
// Dense contraction:   acc(i, j) [= init(i, j)];   acc(i, j) += X(i, k) * Y(k, j) [+ ...];
//                      [D(i, j) = f(acc(i, j), ...)]
// fused in one GPU-mapped nest.  What is checked, on each computation's canonical form (its own
// iteration-domain dimensions, independent of the schedule):
//   * the update's value is its own element plus products of two loads, its store index does not
//     involve the reduction dimension, the first factor of each product does not involve j and
//     the second does not involve i -- so the only loop-carried dependence is the accumulation
//     along k, with distance (0, 0, 1);
//   * iteration domains are boxes; index functions are affine with unit stride along k or i
//     (resp. k or j); the operands are not written in the nest;
//   * an initialisation / epilogue fused into the nest touches the same (i, j) element and has
//     no reduction dimension.
// The nest is then replaced by an MFMA kernel (kernels/gemm_mfma.hip.h) whose epilogue is the
// program's own initialisation + epilogue expression, evaluated once per element of the tile.
// Floating-point sums are reassociated (pairs of k per MFMA step), which is what the 1e-4
// relative tolerance of the parity statement is for; integer-valued data stays exact.
namespace {

struct canon_dim {
    std::string name;   // dimension name in the computation's iteration domain
    std::string cvar;   // "c<p>" in the canonical nest
    expr lo, hi;        // inclusive bounds (undefined when the dimension has a single value)
    bool in_kernel = false;
    std::string kvar;   // name in the emitted kernel
};

struct canon {
    computation *comp = nullptr;
    node_ptr leaf;       // canonical leaf
    node_ptr real;       // leaf in the scheduled program
    std::vector<canon_dim> dims;
    std::map<std::string, expr> subs;  // cvar -> kernel variable / parameter
};

bool canonicalize(function *f, const node_ptr &real, const std::set<std::string> &inner, canon &out) {
    out.comp = real->comp;
    out.real = real;
    node_ptr n = lir::canonical_nest(*f, *real->comp, true);
    const auto &names = real->comp->get_iteration_domain_dimension_names();
    out.dims.resize(names.size());
    for (size_t p = 0; p < names.size(); p++) {
        out.dims[p].name = names[p];
        out.dims[p].cvar = "c" + std::to_string(p);
    }
    while (n && n->kind != node_kind::leaf) {
        if (n->kind == node_kind::loop) {
            int p = std::atoi(n->iterator.c_str() + 1);
            if (p < 0 || p >= (int)out.dims.size()) return false;
            out.dims[p].lo = n->init;
            out.dims[p].hi = n->upper;
            if (!lir::simplify(n->increment).is_integer_literal() || lir::simplify(n->increment).get_int_val() != 1) return false;
            n = n->body;
        } else if (n->kind == node_kind::cond) {
            if (n->else_body) return false;
            n = n->then_body;
        } else if (n->kind == node_kind::block && n->children.size() == 1) {
            n = n->children[0];
        } else {
            return false;
        }
    }
    if (!n) return false;
    out.leaf = n;
    // box: no bound mentions another dimension
    for (auto &d : out.dims)
        for (auto &o : out.dims)
            if (d.lo.is_defined() && (lir::mentions(d.lo, o.cvar) || lir::mentions(d.hi, o.cvar))) return false;
    for (auto &d : out.dims) {
        auto it = real->iterators.find(d.name);
        if (it == real->iterators.end()) return false;
        for (auto &in : inner)
            if (lir::mentions(it->second, in)) d.in_kernel = true;
        // A dimension split between host loops and the kernel: one launch covers part of its
        // range only, which the canonical bounds do not describe.
        bool partly_outside = false;
        if (d.in_kernel)
            it->second.visit([&](const expr &x) {
                if (x.get_expr_type() != e_var || inner.count(x.get_name())) return;
                const std::string &nm = x.get_name();
                if (nm.size() > 1 && nm[0] == 'c' && nm.find_first_not_of("0123456789", 1) == std::string::npos) partly_outside = true;
            });
        if (partly_outside) return false;
    }
    return true;
}

// ---- per-thread accumulators, proven on the schedule ---------------------------------------
//
// A private accumulator (registers, or a per-thread array addressed by tile remainders) ties an
// initialisation, an update and an epilogue together only through the schedule: statement X
// belongs with update instance U[...] when both run in the same thread of the same launch and
// touch the same accumulator element.  The relation is built from the schedules and access
// relations, so the pairing of dimensions does not depend on how the generated loops are named
// or nested (register tiles interchanged below the reduction loop, for instance).

// instance -> values of the loop levels from the outermost down to the innermost thread level
isl_map *thread_of(function *f, computation *c, int &depth) {
    int last = -1;
    for (int l = 0; l < c->get_loop_levels_number(); l++)
        if (f->gpu_thread_position(c->get_name(), l) >= 0) last = l;
    if (last < 0) return nullptr;
    depth = last + 1;
    isl_set *dom = isl_set_copy(c->get_iteration_domain());
    if (f->get_program_context()) dom = isl_set_intersect_params(dom, isl_set_copy(f->get_program_context()));
    isl_map *m = isl_map_intersect_domain(isl_map_copy(c->get_schedule()), dom);
    for (int pos = (int)isl_map_dim(m, isl_dim_out) - 1; pos >= 0; pos--) {
        const bool keep = pos >= 2 && pos % 2 == 0 && (pos - 2) / 2 <= last;
        if (!keep) m = isl_map_project_out(m, isl_dim_out, pos, 1);
    }
    return m;
}

// instance of x -> accumulator element: its own store when x writes the accumulator buffer,
// else the element of the update (or initialisation) instance that its expression reads
isl_map *accumulator_element_of(computation *x, const std::vector<computation *> &writers, const std::string &acc_buffer) {
    if (x->get_access_relation() && acc_buffer == isl_map_get_tuple_name(x->get_access_relation(), isl_dim_out))
        return isl_map_copy(x->get_access_relation());
    for (computation *w : writers) {
        std::vector<expr> args;
        x->get_expr().visit([&](const expr &e) {
            if (args.empty() && e.get_expr_type() == e_op && e.get_op_type() == o_access && e.get_name() == w->get_name()) args = e.get_access();
        });
        if (args.empty() || !w->get_access_relation()) continue;
        std::vector<std::string> to;
        bool ok = true;
        for (auto &a : args) to.push_back(expr_to_isl_str(a, ok));
        if (!ok) return nullptr;
        const std::string text = "{ " + x->get_name() + "[" + join(x->get_iteration_domain_dimension_names(), ", ") + "] -> " +
                                 w->get_name() + "[" + join(to, ", ") + "] }";
        isl_map *m = isl_map_read_from_str(x->get_ctx(), text.c_str());
        if (!m) return nullptr;
        return isl_map_apply_range(m, isl_map_copy(w->get_access_relation()));
    }
    return nullptr;
}

// { x[...] -> u[...] : same thread of the same launch, same accumulator element }
isl_map *same_thread_same_element(function *f, computation *x, computation *u, const std::vector<computation *> &writers,
                                  const std::string &acc_buffer) {
    int dx = 0, du = 0;
    isl_map *tx = thread_of(f, x, dx), *tu = thread_of(f, u, du);
    isl_map *ex = accumulator_element_of(x, writers, acc_buffer), *eu = accumulator_element_of(u, writers, acc_buffer);
    if (!tx || !tu || !ex || !eu || dx != du ||
        isl_map_dim(ex, isl_dim_out) != isl_map_dim(eu, isl_dim_out) ||
        std::string(isl_map_get_tuple_name(ex, isl_dim_out)) != isl_map_get_tuple_name(eu, isl_dim_out)) {
        for (isl_map *m : {tx, tu, ex, eu}) if (m) isl_map_free(m);
        return nullptr;
    }
    return isl_map_apply_range(isl_map_range_product(tx, ex), isl_map_reverse(isl_map_range_product(tu, eu)));
}

bool forces_equal(isl_map *r, int in_pos, int out_pos) {
    isl_map *e = isl_map_equate(isl_map_copy(r), isl_dim_in, in_pos, isl_dim_out, out_pos);
    const bool yes = isl_map_is_subset(r, e) == isl_bool_true;
    isl_map_free(e);
    return yes;
}

// Pairs every in-kernel dimension of x with the dimension of the update that always carries the
// same value in related instances (pairs[q] = p, or -1 for the other dimensions of x).  Fails
// when some in-kernel dimension has no partner, when two share one, or when some update
// instance has no related instance of x.
bool pair_through_accumulator(function *f, const canon &x, const canon &u, const std::vector<computation *> &writers,
                              const std::string &acc_buffer, std::vector<int> &pairs) {
    isl_map *r = same_thread_same_element(f, x.comp, u.comp, writers, acc_buffer);
    if (!r) return false;
    bool ok = isl_map_is_empty(r) == isl_bool_false;
    pairs.assign(x.dims.size(), -1);
    std::set<int> taken;
    for (size_t q = 0; q < x.dims.size() && ok; q++) {
        if (!x.dims[q].in_kernel || !x.dims[q].lo.is_defined()) continue;
        for (size_t p = 0; p < u.dims.size() && pairs[q] < 0; p++)
            if (u.dims[p].in_kernel && u.dims[p].lo.is_defined() && !taken.count((int)p) && forces_equal(r, (int)q, (int)p)) pairs[q] = (int)p;
        if (pairs[q] < 0) ok = false; else taken.insert(pairs[q]);
    }
    if (ok) {
        isl_set *served = isl_map_range(isl_map_copy(r));
        isl_set *all = isl_set_copy(u.comp->get_iteration_domain());
        if (f->get_program_context()) all = isl_set_intersect_params(all, isl_set_copy(f->get_program_context()));
        ok = isl_set_is_subset(all, served) == isl_bool_true;
        isl_set_free(served);
        isl_set_free(all);
    }
    isl_map_free(r);
    return ok;
}

// Within a thread, update instances that share an accumulator element agree on every one of
// the given dimensions: no two results of the thread live in the same element.
bool accumulator_elements_are_private(function *f, const canon &u, const std::vector<int> &spatial, const std::string &acc_buffer) {
    isl_map *r = same_thread_same_element(f, u.comp, u.comp, {u.comp}, acc_buffer);
    if (!r) return false;
    bool ok = true;
    for (int p : spatial) ok = ok && forces_equal(r, p, p);
    isl_map_free(r);
    return ok;
}

void flatten_sum(const expr &e, std::vector<expr> &terms) {
    if (e.get_expr_type() == e_op && e.get_op_type() == o_add) {
        flatten_sum(e.get_operand(0), terms);
        flatten_sum(e.get_operand(1), terms);
    } else {
        terms.push_back(e);
    }
}

bool is_load(const expr &e) { return e.get_expr_type() == e_op && e.get_op_type() == o_access; }

// A factor of a product: a load, possibly widened to fp32 (bf16 storage).
bool is_factor(const expr &e) {
    if (is_load(e)) return true;
    return e.get_expr_type() == e_op && e.get_op_type() == o_cast && e.get_data_type() == p_float32 && is_load(e.get_operand(0));
}
expr strip_cast(const expr &e) { return is_load(e) ? e : e.get_operand(0); }

bool same_element(const expr &load, const buffer *b, const std::vector<expr> &idx) {
    if (!is_load(load) || load.get_name() != b->get_name() || load.get_access().size() != idx.size()) return false;
    for (size_t i = 0; i < idx.size(); i++)
        if (!lir::simplify(load.get_access()[i]).is_equal(lir::simplify(idx[i]))) return false;
    return true;
}

bool reads_buffer(const expr &e, const std::string &bn) {
    bool r = false;
    e.visit([&](const expr &x) { if (is_load(x) && x.get_name() == bn) r = true; });
    return r;
}

struct gemm_operand {
    buffer *buf = nullptr;
    expr base, ld;
    bool kmajor = false;
};

std::string sanitize_id(const std::string &s) {
    std::string r;
    for (char c : s) r += (isalnum((unsigned char)c) ? c : '_');
    return r;
}

bool literal_value(const expr &e, long &v) {
    expr s = lir::simplify(e);
    if (!s.is_integer_literal()) return false;
    v = s.get_int_val();
    return true;
}

// Is the integer expression provably a multiple of m (whatever its variables are)?
bool multiple_of(const expr &e_in, long m) {
    const expr e = lir::simplify(e_in);
    if (e.is_integer_literal()) return e.get_int_val() % m == 0;
    if (e.get_expr_type() != e_op) return false;
    switch (e.get_op_type()) {
    case o_add:
    case o_sub: return multiple_of(e.get_operand(0), m) && multiple_of(e.get_operand(1), m);
    case o_mul: return multiple_of(e.get_operand(0), m) || multiple_of(e.get_operand(1), m);
    case o_minus:
    case o_cast: return multiple_of(e.get_operand(0), m);
    default: return false;
    }
}

// e as constant + sum of coefficient * variable (integers); false when e is not of that form.
bool affine_form(const expr &e_in, std::map<std::string, long> &coef, long &constant, long scale = 1) {
    const expr e = lir::simplify(e_in);
    if (e.is_integer_literal()) { constant += scale * e.get_int_val(); return true; }
    if (e.get_expr_type() == e_var) { coef[e.get_name()] += scale; return true; }
    if (e.get_expr_type() != e_op) return false;
    switch (e.get_op_type()) {
    case o_add: return affine_form(e.get_operand(0), coef, constant, scale) && affine_form(e.get_operand(1), coef, constant, scale);
    case o_sub: return affine_form(e.get_operand(0), coef, constant, scale) && affine_form(e.get_operand(1), coef, constant, -scale);
    case o_minus: return affine_form(e.get_operand(0), coef, constant, -scale);
    case o_cast: return affine_form(e.get_operand(0), coef, constant, scale);
    case o_mul: {
        long v;
        if (literal_value(e.get_operand(0), v)) return affine_form(e.get_operand(1), coef, constant, scale * v);
        if (literal_value(e.get_operand(1), v)) return affine_form(e.get_operand(0), coef, constant, scale * v);
        return false;
    }
    default: return false;
    }
}

// a - b is the same non-zero integer whatever the variables are
bool differ_by_nonzero_constant(const expr &a, const expr &b) {
    std::map<std::string, long> coef;
    long c = 0;
    if (!affine_form(a, coef, c, 1) || !affine_form(b, coef, c, -1)) return false;
    for (auto &kv : coef)
        if (kv.second != 0) return false;
    return c != 0;
}

bool same_affine_value(const expr &a, const expr &b) {
    std::map<std::string, long> coef;
    long c = 0;
    if (!affine_form(a, coef, c, 1) || !affine_form(b, coef, c, -1)) return lir::simplify(a).is_equal(lir::simplify(b));
    for (auto &kv : coef)
        if (kv.second != 0) return false;
    return c == 0;
}

bool reject(int where) {
    if (std::getenv("TIRAMISU_HIP_REPORT")) std::cout << "[tiramisu-hip] contraction check " << where << " failed" << std::endl;
    return false;
}

}  // namespace

bool emit_contraction(context &ctx, const node_ptr &root, launch_plan &plan, const fusion_request *fuse) {
    if (backend_option("TIRAMISU_NO_MFMA")) return false;
    const bool with_consumer = fuse && fuse->consumer && !backend_option("TIRAMISU_MFMA_NO_CONSUMER");
    const bool batched = fuse && !fuse->batch_iterator.empty();
    if (fuse && fuse->consumer && !with_consumer) return false;
    function *f = ctx.f;
    std::set<std::string> inner;
    std::vector<node_ptr> leaves;
    // LDS tiles that the schedule installed with cache_shared(): their declaration, cooperative
    // copy and barriers are left out, and the computation they serve is analysed as written,
    // once each tile is proven to hold what the computation reads through it.
    std::set<computation *> cached;
    bool bad = false;
    lir::walk(root, [&](const node_ptr &x) {
        if (x->kind == node_kind::loop) inner.insert(x->iterator);
        if (x->kind != node_kind::leaf) return;
        if (x->comp && x->comp->get_cache_consumer()) { cached.insert(x->comp->get_cache_consumer()); return; }
        if (x->lkind == leaf_kind::allocate || x->lkind == leaf_kind::release) {
            if (x->target->get_location() == memory_location::global || x->target->get_location() == memory_location::host) bad = true;
            return;
        }
        if (x->lkind != leaf_kind::assign || x->predicate.is_defined() || !x->lets.empty()) bad = true;
        leaves.push_back(x);
    });
    if (bad || leaves.empty() || leaves.size() > 3) return reject(2);
    for (computation *c : cached) {
        bool in_nest = false;
        for (auto &l : leaves) in_nest |= l->comp == c;
        if (!in_nest || !c->shared_caches_cover_reads()) return reject(26);
    }
    for (auto &l : leaves)   // every tile of a cached computation must have been seen in this nest
        if (!l->comp->get_shared_caches().empty() && !cached.count(l->comp)) return reject(26);

    // ---- find the update: own element + products of loads
    int ui = -1;
    std::vector<canon> cs(leaves.size());
    for (size_t l = 0; l < leaves.size(); l++)
        if (!canonicalize(f, leaves[l], inner, cs[l])) return reject(3);
    std::vector<std::pair<expr, expr>> products;
    for (size_t l = 0; l < leaves.size() && ui < 0; l++) {
        const node_ptr &cl = cs[l].leaf;
        if (!cl->lhs || cl->rhs.get_data_type() != p_float32) continue;
        std::vector<expr> terms;
        flatten_sum(cl->rhs, terms);
        int self = 0;
        std::vector<std::pair<expr, expr>> prods;
        bool shape = true;
        for (auto &t : terms) {
            if (same_element(t, cl->lhs, cl->lhs_index)) { self++; continue; }
            if (t.get_expr_type() == e_op && t.get_op_type() == o_mul && is_factor(t.get_operand(0)) && is_factor(t.get_operand(1)))
                prods.push_back({strip_cast(t.get_operand(0)), strip_cast(t.get_operand(1))});
            else
                shape = false;
        }
        if (shape && self == 1 && !prods.empty()) { ui = (int)l; products = prods; }
    }
    if (ui < 0) return reject(4);
    canon &U = cs[ui];
    const node_ptr ureal = leaves[ui];
    const int ii = ui - 1, ei = ui + 1;   // optional initialisation before, epilogue after
    if (ii > 0 || ei < (int)leaves.size() - 1) return reject(5);
    const bool has_init = ii == 0, has_epi = ei == (int)leaves.size() - 1 && ei > ui;

    // ---- dimensions of the update.  A spatial dimension is one that the accumulator's store
    // index involves or, for a per-thread accumulator (whose index is constant or a tile
    // remainder), one that the fused initialisation / epilogue also iterates: same expression
    // of the loop iterators in the scheduled program.  The remaining in-kernel dimensions are
    // reduction dimensions.
    const buffer *acc_buf = ureal->lhs;
    const bool acc_private = acc_buf->get_location() == memory_location::reg || acc_buf->get_location() == memory_location::local;
    if (!acc_private && acc_buf->get_location() != memory_location::global) return reject(15);
    if (!has_init && acc_private) return reject(16);   // a private accumulator must be initialised in the nest
    std::vector<int> spatial, reduction;
    for (size_t p = 0; p < U.dims.size(); p++) {
        if (!U.dims[p].in_kernel || !U.dims[p].lo.is_defined()) continue;
        bool is_spatial = false;
        if (!acc_private) {
            for (auto &ix : U.leaf->lhs_index)
                if (lir::mentions(ix, U.dims[p].cvar)) is_spatial = true;
        } else {
            const expr mine = lir::simplify(ureal->iterators.at(U.dims[p].name));
            for (int other : {ii, ei}) {
                if (other < 0 || other >= (int)leaves.size() || other == ui) continue;
                for (auto &d : cs[other].dims)
                    if (d.in_kernel && d.lo.is_defined() && lir::simplify(leaves[other]->iterators.at(d.name)).is_equal(mine)) is_spatial = true;
            }
        }
        (is_spatial ? spatial : reduction).push_back((int)p);
    }
    // register tiles nested differently in the fused statements: pair dimensions on the schedule instead
    std::map<int, std::vector<int>> paired;   // leaf index -> dimension of that leaf -> dimension of the update
    if (acc_private && has_init && (spatial.size() < 2 || reduction.empty())) {
        std::vector<computation *> writers = {U.comp, cs[ii].comp};
        const std::string acc_name = acc_buf->get_name();
        std::vector<int> pi;
        if (!pair_through_accumulator(f, cs[ii], U, writers, acc_name, pi)) return reject(6);
        spatial.clear();
        reduction.clear();
        std::set<int> sp;
        for (int p : pi) if (p >= 0) sp.insert(p);
        for (size_t p = 0; p < U.dims.size(); p++)
            if (U.dims[p].in_kernel && U.dims[p].lo.is_defined()) (sp.count((int)p) ? spatial : reduction).push_back((int)p);
        if (!accumulator_elements_are_private(f, U, spatial, acc_name)) return reject(6);
        paired[ii] = pi;
        const int ei_ = ui + 1;
        if (ei_ < (int)leaves.size()) {
            std::vector<int> pe;
            if (!pair_through_accumulator(f, cs[ei_], U, writers, acc_name, pe)) return reject(6);
            paired[ei_] = pe;
        }
    }
    if (spatial.size() < 2 || reduction.empty()) return reject(6);

    // ---- the GEMM view: N dimensions are the spatial dimensions of the factor that involves the
    // innermost spatial dimension, M dimensions are the others; every product must have one
    // factor over (M, K) and one over (K, N)
    auto dims_of = [&](const expr &load, const std::vector<int> &among) {
        std::set<int> r;
        for (int p : among)
            for (auto &ix : load.get_access())
                if (lir::mentions(ix, U.dims[p].cvar)) r.insert(p);
        return r;
    };
    const int innermost = spatial.back();
    std::set<int> Nset;
    for (auto &pr : products)
        for (const expr *ld : {&pr.first, &pr.second}) {
            std::set<int> d = dims_of(*ld, spatial);
            if (d.count(innermost)) { if (Nset.empty()) Nset = d; else if (Nset != d) return reject(7); }
        }
    if (Nset.empty()) return reject(7);
    std::vector<int> Mg, Ng, Kg = reduction;
    for (int p : spatial) (Nset.count(p) ? Ng : Mg).push_back(p);
    if (Mg.empty()) return reject(8);
    for (auto &pr : products) {
        std::set<int> dx = dims_of(pr.first, spatial), dy = dims_of(pr.second, spatial);
        std::set<int> Mset(Mg.begin(), Mg.end());
        if (dx == Nset && dy == Mset) std::swap(pr.first, pr.second);   // written as Y * X
        else if (!(dx == Mset && dy == Nset)) return reject(8);
    }

    // ---- kernel names.  Outer dimensions become scalar parameters whose value the host computes;
    // in-kernel dimensions become _d<p>, recovered from the flattened row / column / k index.
    struct outer_param { std::string name; expr host_value; };
    std::vector<outer_param> outers;
    auto name_outer_dims = [&](canon &c) {
        for (size_t p = 0; p < c.dims.size(); p++) {
            canon_dim &d = c.dims[p];
            if (d.in_kernel || !d.lo.is_defined()) continue;
            d.kvar = "_o_" + sanitize_id(c.comp->get_name()) + "_" + std::to_string(p);
            outers.push_back({d.kvar, c.real->iterators.at(d.name)});
            c.subs[d.cvar] = var(d.kvar);
        }
    };
    name_outer_dims(U);
    for (int p : spatial) { U.dims[p].kvar = "_d" + std::to_string(p); U.subs[U.dims[p].cvar] = var(U.dims[p].kvar); }
    for (int p : reduction) { U.dims[p].kvar = "_d" + std::to_string(p); U.subs[U.dims[p].cvar] = var(U.dims[p].kvar); }

    // initialisation / epilogue: their in-kernel dimensions must be spatial dimensions of the update
    auto bind_to_update = [&](canon &c) -> bool {
        const std::vector<int> *proven = nullptr;
        for (auto &pr : paired)
            if (&cs[pr.first] == &c) proven = &pr.second;
        for (size_t p = 0; p < c.dims.size(); p++) {
            canon_dim &d = c.dims[p];
            if (!d.lo.is_defined() || !d.in_kernel) continue;
            const expr mine = lir::simplify(c.real->iterators.at(d.name));
            int match = -1;
            if (proven) match = (*proven)[p];
            else
                for (int sp : spatial)
                    if (mine.is_equal(lir::simplify(ureal->iterators.at(U.dims[sp].name)))) match = sp;
            if (match < 0) return false;
            if (!lir::simplify(d.lo).is_equal(lir::simplify(U.dims[match].lo)) || !lir::simplify(d.hi).is_equal(lir::simplify(U.dims[match].hi)))
                return false;
            c.subs[d.cvar] = var(U.dims[match].kvar);
        }
        name_outer_dims(c);
        return true;
    };
    if (has_init && !bind_to_update(cs[ii])) return reject(11);
    if (has_epi && !bind_to_update(cs[ei])) return reject(12);
    const buffer *out_buf = has_epi ? cs[ei].leaf->lhs : U.leaf->lhs;
    if (!out_buf) return reject(7);

    // the accumulator element is the same in all fused statements (compared in the scheduled program)
    if (has_init && (leaves[ii]->lhs != acc_buf ||
                     (paired.empty() && !same_element(expr(o_access, acc_buf->get_name(), leaves[ii]->lhs_index, p_float32), acc_buf, ureal->lhs_index))))
        return reject(13);
    if (has_init && reads_buffer(cs[ii].leaf->rhs, acc_buf->get_name())) return reject(14);
    // The kernel's epilogue has one value at hand per element: the finished sum of that element.  A fused
    // statement may therefore read the accumulator and the output only at the element it belongs to (index
    // compared in kernel variables; for a private accumulator the pairing above already ties the elements).
    auto reads_only = [&](canon &c, const buffer *b, const std::vector<expr> &own, const std::map<std::string, expr> &own_subs) {
        bool only = true;
        c.leaf->rhs.visit([&](const expr &x) {
            if (!is_load(x) || x.get_name() != b->get_name()) return;
            if (x.get_access().size() != own.size()) { only = false; return; }
            for (size_t d = 0; d < own.size(); d++)
                if (!lir::simplify(x.get_access()[d].substitute(c.subs)).is_equal(lir::simplify(own[d].substitute(own_subs)))) only = false;
        });
        return only;
    };
    if (has_epi && paired.empty() && !reads_only(cs[ei], acc_buf, U.leaf->lhs_index, U.subs)) return reject(27);
    if (has_epi && out_buf != acc_buf)
        for (int other : {ii, ei})
            if (other >= 0 && other < (int)leaves.size() && other != ui && !reads_only(cs[other], out_buf, cs[ei].leaf->lhs_index, cs[ei].subs)) return reject(27);

    // ---- extents of the three groups
    struct group_info { std::vector<int> dims; std::vector<expr> extent; bool literal = true; std::vector<long> ext; expr total; };
    auto make_group = [&](const std::vector<int> &dims) {
        group_info g;
        g.dims = dims;
        for (int p : dims) {
            expr e = lir::simplify(lir::simplify(U.dims[p].hi - U.dims[p].lo) + 1).substitute(U.subs);
            g.extent.push_back(e);
            long v;
            if (literal_value(e, v)) g.ext.push_back(v); else { g.ext.push_back(-1); g.literal = false; }
            g.total = g.total.is_defined() ? lir::simplify(g.total * e) : e;
        }
        return g;
    };
    group_info GM = make_group(Mg), GN = make_group(Ng), GK = make_group(Kg);
    for (const group_info *g : {&GM, &GN, &GK})
        if (g->dims.size() > 1 && !g->literal) return reject(9);   // several dimensions flatten only with constant extents

    // ---- operands: offset of element (row digits, k digits) = base + sum coef_p * (d_p - lo_p)
    struct operand_info {
        buffer *buf = nullptr;
        expr base;
        std::map<int, expr> coef;        // per in-kernel dimension
        bool linear = false, kmajor = false;
        expr ld;
        bool gather_vec = false;         // gather: 4 consecutive elements are contiguous
        bool gather_kdir = false;        // gather: vector direction is k
    };
    std::map<std::string, expr> at_origin = U.subs;
    for (int p : spatial) at_origin[U.dims[p].cvar] = U.dims[p].lo;
    for (int p : reduction) at_origin[U.dims[p].cvar] = U.dims[p].lo;
    std::set<std::string> written = {acc_buf->get_name(), out_buf->get_name()};
    // linear: offsets along the group are stride * flattened index
    auto group_stride = [&](const operand_info &o, const group_info &g, expr &stride) -> bool {
        stride = o.coef.at(g.dims.back());
        if (g.dims.size() == 1) return true;
        long sv;
        if (!literal_value(stride, sv)) return false;
        long mult = sv;
        for (int q = (int)g.dims.size() - 1; q >= 0; q--) {
            long cv;
            if (!literal_value(o.coef.at(g.dims[q]), cv) || cv != mult) return false;
            mult *= g.ext[q];
        }
        return true;
    };
    auto analyse = [&](const expr &ld, const group_info &rowg, operand_info &o) -> bool {
        buffer *b = f->get_buffers().at(ld.get_name());
        if (b->get_location() != memory_location::global || written.count(b->get_name())) return false;
        if (b->get_elements_type() != p_float32 && b->get_elements_type() != p_bfloat16) return false;
        o.buf = b;
        expr lin = lir::linearize(b, ld.get_access());
        bool okc = true;
        for (const group_info *g : std::vector<const group_info *>{&rowg, &GK})
            for (int p : g->dims) o.coef[p] = lir::simplify(lir::coefficient(lin, U.dims[p].cvar, okc).substitute(U.subs));
        if (!okc) return false;
        o.base = lir::simplify(lin.substitute(at_origin));
        expr rs, ks;
        long v;
        const bool rl = group_stride(o, rowg, rs), kl = group_stride(o, GK, ks);
        if (rl && kl && literal_value(ks, v) && v == 1) { o.linear = true; o.kmajor = true; o.ld = rs; return true; }
        if (rl && kl && literal_value(rs, v) && v == 1) { o.linear = true; o.kmajor = false; o.ld = ks; return true; }
        // gather: every coefficient must be a constant
        for (auto &kv : o.coef)
            if (!literal_value(kv.second, v)) return false;
        if (!rowg.literal || !GK.literal) return false;
        long cr, ck;
        literal_value(o.coef.at(rowg.dims.back()), cr);
        literal_value(o.coef.at(GK.dims.back()), ck);
        if (ck == 1 && GK.ext.back() % 4 == 0) { o.gather_vec = true; o.gather_kdir = true; o.kmajor = true; }
        else if (cr == 1 && rowg.ext.back() % 4 == 0) { o.gather_vec = true; o.gather_kdir = false; o.kmajor = false; }
        else { o.gather_vec = false; o.kmajor = false; }
        return true;
    };
    std::vector<std::pair<operand_info, operand_info>> operands;
    for (auto &pr : products) {
        operand_info a, b;
        if (!analyse(pr.first, GM, a) || !analyse(pr.second, GN, b)) return reject(17);
        operands.push_back({a, b});
    }
    for (auto &o : operands)
        if (o.first.kmajor != operands[0].first.kmajor || o.second.kmajor != operands[0].second.kmajor) return reject(20);
    // storage type: all fp32, or all bf16 (plain row-major operands only)
    bool bf16 = false;
    {
        int nb = 0, nf = 0;
        for (auto &o : operands)
            for (const operand_info *g : {&o.first, &o.second}) (g->buf->get_elements_type() == p_bfloat16 ? nb : nf)++;
        if (nb && nf) return reject(23);
        bf16 = nb > 0;
    }

    // ---- sizes and tile configuration
    const expr Me = GM.total, Ne = GN.total, Ke = GK.total;
    long Ml = -1, Nl = -1, Kl = -1;
    const bool lit = literal_value(Me, Ml) && literal_value(Ne, Nl) && literal_value(Ke, Kl);

    // ---- a point-wise consumer nest folded into the kernel (see fusion_request).  Its statements are
    // written per point (row, unit) of a two-dimensional domain; the row is the contraction's M index,
    // and the result is read only at columns unit + q * units of that row.
    std::vector<canon> xs;               // consumer statements, in program order
    std::vector<node_ptr> xleaves;
    int G = 1;                           // column groups of the result
    long UE = 0, u_lo = 0;               // units per group, first unit
    std::vector<std::map<std::string, int>> acc_group;   // per statement: printed canonical load of the result -> group q
    std::vector<int> row_of, unit_of;    // per statement: which of its dimensions is the row / the unit
    if (with_consumer) {
        if (has_epi || acc_private || Mg.size() != 1 || Ng.size() != 1 || !lit || bf16) return reject(30);
        std::set<std::string> xinner;
        bool xbad = false;
        lir::walk(fuse->consumer, [&](const node_ptr &x) {
            if (x->kind == node_kind::cond) xbad = true;
            if (x->kind == node_kind::loop) {
                xinner.insert(x->iterator);
                if (x->gpu_block < 0 && x->gpu_thread < 0) xbad = true;   // one point per thread: a point's statements are the leaves in order
            }
            if (x->kind != node_kind::leaf) return;
            if (x->lkind != leaf_kind::assign || x->predicate.is_defined() || !x->lets.empty() || !x->lhs) xbad = true;
            xleaves.push_back(x);
        });
        if (xbad || xleaves.empty()) return reject(30);
        xs.resize(xleaves.size());
        for (size_t n = 0; n < xleaves.size(); n++)
            if (!canonicalize(f, xleaves[n], xinner, xs[n])) return reject(30);
        const canon_dim &UM = U.dims[Mg[0]], &UN = U.dims[Ng[0]];
        long m_lo, m_hi, n_lo, n_hi;
        if (!literal_value(UM.lo, m_lo) || !literal_value(UM.hi, m_hi) || !literal_value(UN.lo, n_lo) || !literal_value(UN.hi, n_hi)) return reject(30);
        // host value of an index expression of statement c: dimensions outside the kernel by their value in
        // terms of the host loops, dimensions inside renamed per side so that they never cancel
        auto host_view = [&](const canon &c, const expr &e, const std::string &side) {
            std::map<std::string, expr> m;
            for (auto &d : c.dims) {
                if (!d.lo.is_defined()) continue;
                if (d.in_kernel) m[d.cvar] = var(side + d.cvar);
                else m[d.cvar] = c.real->iterators.at(d.name);
            }
            return lir::simplify(e.substitute(m));
        };
        // a dimension in which the two elements always differ by a non-zero constant
        auto always_apart = [&](const canon &a, const std::vector<expr> &ia, const canon &b, const std::vector<expr> &ib) {
            if (ia.size() != ib.size()) return false;
            for (size_t d = 0; d < ia.size(); d++) {
                if (differ_by_nonzero_constant(host_view(a, ia[d], "_a_"), host_view(b, ib[d], "_b_"))) return true;
            }
            return false;
        };
        // roles of the two dimensions, from the first statement that reads the result
        expr Er, Eu;   // row / unit as expressions of the consumer nest's loop iterators
        row_of.assign(xs.size(), -1);
        unit_of.assign(xs.size(), -1);
        auto in_kernel_dims = [&](const canon &c) {
            std::vector<int> r;
            for (size_t p = 0; p < c.dims.size(); p++)
                if (c.dims[p].in_kernel && c.dims[p].lo.is_defined()) r.push_back((int)p);
            return r;
        };
        // matches a load of the result in statement c: row dimension, unit dimension and column offset
        auto match_result_load = [&](const canon &c, const expr &ld, int &pr, int &pu, long &off) {
            if (ld.get_access().size() != U.leaf->lhs_index.size()) return false;
            pr = pu = -1;
            off = 0;
            for (size_t d = 0; d < U.leaf->lhs_index.size(); d++) {
                const expr ui = lir::simplify(U.leaf->lhs_index[d]), xi = lir::simplify(ld.get_access()[d]);
                const bool in_m = lir::mentions(ui, UM.cvar), in_n = lir::mentions(ui, UN.cvar);
                if (in_m || in_n) {
                    if (ui.get_expr_type() != e_var) return false;           // the result's index is the bare dimension
                    bool found = false;
                    for (int p : in_kernel_dims(c)) {
                        long o;
                        if (!var_plus_const(xi, c.dims[p].cvar, o)) continue;
                        if (in_m) { if (o != 0) return false; pr = p; } else { pu = p; off = o; }
                        found = true;
                    }
                    if (!found) return false;
                } else {
                    for (int p : in_kernel_dims(c)) if (lir::mentions(xi, c.dims[p].cvar)) return false;
                    if (!same_affine_value(host_view(U, ui, "_a_"), host_view(c, xi, "_b_"))) return false;
                }
            }
            return pr >= 0 && pu >= 0 && pr != pu;
        };
        for (size_t n = 0; n < xs.size() && !Er.is_defined(); n++) {
            expr first;
            xs[n].leaf->rhs.visit([&](const expr &x) { if (!first.is_defined() && is_load(x) && x.get_name() == acc_buf->get_name()) first = x; });
            if (!first.is_defined()) continue;
            int pr, pu;
            long off;
            if (!match_result_load(xs[n], first, pr, pu, off)) return reject(31);
            Er = lir::simplify(xleaves[n]->iterators.at(xs[n].dims[pr].name));
            Eu = lir::simplify(xleaves[n]->iterators.at(xs[n].dims[pu].name));
            long lo, hi;
            if (!literal_value(xs[n].dims[pu].lo, lo) || !literal_value(xs[n].dims[pu].hi, hi)) return reject(31);
            u_lo = lo;
            UE = hi - lo + 1;
        }
        if (!Er.is_defined() || UE <= 0 || (n_hi - n_lo + 1) % UE != 0) return reject(31);
        G = (int)((n_hi - n_lo + 1) / UE);
        acc_group.resize(xs.size());
        for (size_t n = 0; n < xs.size(); n++) {
            canon &X = xs[n];
            const std::vector<int> ik = in_kernel_dims(X);
            if (ik.size() != 2) return reject(32);
            for (int p : ik) {
                const expr e = lir::simplify(xleaves[n]->iterators.at(X.dims[p].name));
                long lo, hi;
                if (!literal_value(X.dims[p].lo, lo) || !literal_value(X.dims[p].hi, hi)) return reject(32);
                if (e.is_equal(Er) && lo == m_lo && hi == m_hi) row_of[n] = p;
                else if (e.is_equal(Eu) && lo == u_lo && hi - lo + 1 == UE) unit_of[n] = p;
                else return reject(32);
            }
            if (row_of[n] < 0 || unit_of[n] < 0) return reject(32);
            // the result is read only at (own row, own unit + q * units)
            bool okx = true;
            X.leaf->rhs.visit([&](const expr &x) {
                if (!is_load(x) || x.get_name() != acc_buf->get_name()) return;
                int pr, pu;
                long off;
                if (!match_result_load(X, x, pr, pu, off) || pr != row_of[n] || pu != unit_of[n]) { okx = false; return; }
                const long shifted = off + u_lo - n_lo;
                if (shifted < 0 || shifted % UE != 0 || shifted / UE >= G) { okx = false; return; }
                acc_group[n][x.to_str()] = (int)(shifted / UE);
            });
            if (!okx) return reject(33);
            // it may not write what the contraction reads or writes in the same launch ...
            if (X.leaf->lhs == acc_buf || X.leaf->lhs == out_buf) return reject(34);
            auto clashes = [&](const canon &reader, const expr &e) {
                bool clash = false;
                e.visit([&](const expr &x) {
                    if (is_load(x) && x.get_name() == X.leaf->lhs->get_name() && !always_apart(X, X.leaf->lhs_index, reader, x.get_access())) clash = true;
                });
                return clash;
            };
            for (auto &pr : products)
                if (clashes(U, pr.first) || clashes(U, pr.second)) return reject(34);
            if (has_init && clashes(cs[ii], cs[ii].leaf->rhs)) return reject(34);
            // ... and what it reads of the consumer's own buffers is either the element this point wrote
            // (same index text as the point's latest store, checked when the statements are printed) or an
            // element that no point of the launch writes
            X.subs[X.dims[row_of[n]].cvar] = var(UM.kvar);
            X.subs[X.dims[unit_of[n]].cvar] = var("_u");
            name_outer_dims(X);
        }
    }
    int BM = 64, BN = 64, BK = 16, PADX = 1, WGM = 2, WGN = 2, WGK = 1, DEPTH = 1;
    if (lit) {
        if (Ml <= 64 && Nl >= 256 * 256) { BM = 64; BN = 256; WGM = 1; WGN = 4; }   // short, very wide (convolutions)
        else {
            // square tiles: the one whose launch is modelled fastest on this machine (kernels/target_gfx950.h);
            // 192 is what makes 3072 = 16 x 192 one tile per compute unit
            BM = BN = ttarget::square_tile_for(Ml, Nl);
            PADX = BM == 256 ? 0 : 1;
        }
    }
    if (BM == 64 && BN == 64) BK = 32;   // one 32x32 tile per wavefront: longer slices, fewer barriers per flop
    // few C tiles but a long reduction (a batch-sized M against wide weights, as in recurrent cells):
    // 64x32 tiles, and 8 groups of wavefronts share the K range of each tile
    if (lit && !bf16 && BM == 64 && BN == 64 && Ml <= 64 && ((Nl + 63) / 64) <= ttarget::COMPUTE_UNITS / 4 && Nl % 32 == 0 && Kl % 128 == 0 && Kl >= 256 &&
        !backend_option("TIRAMISU_MFMA_NO_SPLITK")) {
        BN = 32; BK = 128; WGM = 2; WGN = 1; WGK = 8; PADX = 0;
        DEPTH = (int)std::min<long>(4, std::max<long>(1, Kl / BK - 1));   // latency-bound: ask for (up to) all slices at once
        // a reduction of 1024 or more (several terms run as one loop): the loop is long enough to hide its own
        // latencies, and four groups of wavefronts with 64-k slices and no extra slices in flight are faster
        // (4-layer LSTM cell, 64x2048x1024 per layer: 1.30 ms per pass against 1.55 ms)
        if ((long)products.size() * Kl >= 1024) { BK = 64; WGK = 4; DEPTH = 1; }
    }
    // at most one 64x64 tile per compute unit and a long reduction: two groups of wavefronts share each
    // (64-k) slice, so that every SIMD has two wavefronts to alternate between (1024^3: 20.6 us against 21.9)
    if (lit && !bf16 && BM == 64 && BN == 64 && WGK == 1 && Ml % 64 == 0 && Nl % 64 == 0 && Kl % 64 == 0 && Kl >= 512 &&
        (Ml / 64) * (Nl / 64) <= ttarget::COMPUTE_UNITS) {
        WGK = 2; BK = 64;
    }
    // a forced square tile starts from that tile's own defaults (no K groups, slices of 32 for 64x64, of 16 above)
    if (const char *e = backend_option("TIRAMISU_MFMA_TILE")) { BM = BN = std::atoi(e); PADX = BM == 256 ? 0 : 1; WGM = WGN = 2; WGK = 1; DEPTH = 1; BK = BM == 64 ? 32 : 16; }
    if (const char *e = backend_option("TIRAMISU_MFMA_BM")) BM = std::atoi(e);
    if (const char *e = backend_option("TIRAMISU_MFMA_BN")) BN = std::atoi(e);
    if (const char *e = backend_option("TIRAMISU_MFMA_WGM")) WGM = std::atoi(e);
    if (const char *e = backend_option("TIRAMISU_MFMA_WGN")) WGN = std::atoi(e);
    if (const char *e = backend_option("TIRAMISU_MFMA_BK")) BK = std::atoi(e);
    if (const char *e = backend_option("TIRAMISU_MFMA_DEPTH")) DEPTH = std::atoi(e);
    if (const char *e = backend_option("TIRAMISU_MFMA_PAD")) PADX = std::atoi(e);
    if (const char *e = backend_option("TIRAMISU_MFMA_WGK")) WGK = std::atoi(e);
    bool bf16_edge = false;
    if (bf16) {
        // 256x256 when that fills the chip, else 128x128 (both load their slices straight into LDS and want whole
        // tiles, 16-byte aligned rows and operands below 2 GiB), else 64x64 -- with guarded loads when tiles hang
        // over the problem, sizes are known at run time only, or rows are not aligned
        for (auto &o : operands)
            if (!o.first.linear || !o.second.linear || !o.first.kmajor || o.second.kmajor) return reject(25);
        bool aligned = true, small_enough = true;
        for (auto &o : operands) {
            long v;
            for (const operand_info *g : {&o.first, &o.second})
                if (!literal_value(g->ld, v) || v % 8 != 0 || !multiple_of(g->base, 8)) aligned = false;
            long lda = 0, ldb = 0;
            if (lit && literal_value(o.first.ld, lda) && literal_value(o.second.ld, ldb)) {
                if ((double)Ml * lda * 2 >= 2147483648.0 || (double)Kl * ldb * 2 >= 2147483648.0) small_enough = false;
            } else {
                small_enough = false;
            }
        }
        WGM = WGN = 2;
        if (lit && aligned && small_enough && (Ml / 256) * (Nl / 256) >= 3 * ttarget::COMPUTE_UNITS / 4 && Ml % 256 == 0 && Nl % 256 == 0 && Kl % 32 == 0) { BM = BN = 256; BK = 32; }
        else if (lit && aligned && small_enough && Ml % 128 == 0 && Nl % 128 == 0 && Kl % 32 == 0 && (Ml / 128) * (Nl / 128) >= 3 * ttarget::COMPUTE_UNITS / 16) { BM = BN = 128; BK = 32; }
        else {
            BM = BN = 64;
            BK = 64;
            bf16_edge = !(lit && aligned && Ml % 64 == 0 && Nl % 64 == 0 && Kl % 64 == 0);
        }
    }
    bool edge = !(lit && Ml % BM == 0 && Nl % BN == 0 && Kl % BK == 0);
    if (bf16) edge = bf16_edge;
    for (auto &o : operands)
        for (const operand_info *g : {&o.first, &o.second}) {
            long v;
            if (g->linear && (!literal_value(g->ld, v) || v % 4 != 0)) edge = true;
            if (g->linear && !multiple_of(g->base, 4)) edge = true;
        }

    // a consumer needs tiles that hold all column groups of their units
    int UB = 0;
    if (with_consumer) {
        UB = BN / G;
        if (BN % G != 0 || UB == 0 || UE % UB != 0 || Nl % BN != 0) return reject(35);
        for (auto &o : operands)
            if (!o.second.linear || (!o.second.kmajor && UB % 4 != 0)) return reject(35);
    }

    // ---- a gathered B operand that is a sliding window (the implicit GEMM of a convolution): k = (channel,
    // taps...) with the channel outermost, offset = f(position) + channel * stride + tap offset.  When the piece
    // of memory that a tile's positions and all taps touch per channel is short, blocks of channels are staged
    // in LDS and the operand is read from there (kernels/gemm_mfma_window.hip.h); else the gather stays as it is.
    bool windowed = false;
    int win_cb = 0, win_taps = 0, win_floats = 0;
    long win_chan_stride = 0, win_channels = 0, win_x_elements = 0;
    std::vector<long> win_tap_offsets;
    int win_splits = 1;                  // pieces that each tile of the last, incomplete round is cut into
    long win_grid = 0, win_scratch_floats = 0, win_counters = 0;
    int win_resident = 1;                // workgroups that share a compute unit
    std::string window_call_head;
    if (!bf16 && !with_consumer && lit && operands.size() == 1 && operands[0].first.linear && operands[0].first.kmajor &&
        !operands[0].second.linear && GK.dims.size() >= 2 && GK.literal && GN.literal && Ml % BM == 0 && Nl % BN == 0 && WGK == 1 &&
        !backend_option("TIRAMISU_MFMA_NO_WINDOW")) {
        const operand_info &xo = operands[0].second;
        std::vector<long> ck, cn;
        bool ok = true;
        long v;
        for (int p : GK.dims) { ok = ok && literal_value(xo.coef.at(p), v); ck.push_back(v); }
        for (int p : GN.dims) { ok = ok && literal_value(xo.coef.at(p), v); cn.push_back(v); }
        long base_lit = 0, lda_lit = 0, abase_lit = 0;
        ok = ok && literal_value(xo.base, base_lit) && base_lit % 4 == 0 && literal_value(operands[0].first.ld, lda_lit) && lda_lit % 4 == 0 &&
             literal_value(operands[0].first.base, abase_lit) && abase_lit % 4 == 0 && xo.buf->has_constant_extents();
        if (ok && ck[0] % 4 == 0 && ck[0] > 0) {
            win_channels = GK.ext[0];
            win_chan_stride = ck[0];
            win_taps = 1;
            for (size_t d = 1; d < GK.dims.size(); d++) win_taps *= (int)GK.ext[d];
            for (int t = 0; t < win_taps; t++) {
                long off = 0, rest = t;
                for (int d = (int)GK.dims.size() - 1; d >= 1; d--) { off += (rest % GK.ext[d]) * ck[d]; rest /= GK.ext[d]; }
                if (off < 0) ok = false;
                win_tap_offsets.push_back(off);
            }
            auto position_offset = [&](long pflat) {
                long off = 0, rest = pflat;
                for (int d = (int)GN.dims.size() - 1; d >= 0; d--) { off += (rest % GN.ext[d]) * cn[d]; rest /= GN.ext[d]; }
                return off;
            };
            long need = 0;
            const long max_tap = *std::max_element(win_tap_offsets.begin(), win_tap_offsets.end());
            for (long n0 = 0; n0 < Nl && ok; n0 += BN) {
                const long f0 = position_offset(n0) & ~3L;
                for (long pp = n0; pp < n0 + BN; pp++) {
                    const long fpos = position_offset(pp);
                    if (fpos < f0) ok = false;              // positions must not run backwards within a tile
                    need = std::max(need, fpos + max_tap - f0 + 1);
                }
            }
            const int cb_max = env_int("TIRAMISU_MFMA_WINDOW_CB", 8);
            for (int cb : {8, 4, 2})
                if (win_cb == 0 && cb <= cb_max && win_channels % cb == 0 && (cb * win_taps) % 4 == 0) win_cb = cb;
            win_floats = (int)((need + 31) / 64 * 64 + 32);      // = 32 mod 64: the two halves of a wavefront on disjoint banks
            if (win_floats < need) win_floats += 64;
            long cnt = 1;
            for (auto &d : xo.buf->get_dim_sizes()) cnt *= lir::simplify(d).get_int_val();
            win_x_elements = cnt - base_lit;
            const long stage_bytes = ((long)win_cb * (win_taps * BM + 32) + (long)win_cb * win_floats) * 4;
            windowed = ok && win_cb > 0 && win_taps <= 64 && (win_taps * BM) % 64 == 0 && 2 * stage_bytes + 64 <= ttarget::LDS_BYTES_PER_CU && cnt < 2147483648L;
            if (windowed) {
                // as many workgroups as the chip holds take tiles from a queue; the tiles left over after the last
                // full round of the grid are cut along the channel blocks into short pieces that fill the end
                const long tiles = (Ml / BM) * (Nl / BN), blocks = win_channels / win_cb;
                // two workgroups per compute unit when their LDS fits: one's tile boundaries (epilogue stores, the wait
                // for the first block) are covered by the other's matrix instructions
                win_resident = 2 * (2 * stage_bytes + 64) <= ttarget::LDS_BYTES_PER_CU ? env_int("TIRAMISU_MFMA_WINDOW_RESIDENT", 2) : 1;
                win_grid = std::min<long>(tiles, (long)ttarget::COMPUTE_UNITS * win_resident);
                const long rest = tiles % win_grid;
                if (rest > 0 && tiles > win_grid && !backend_option("TIRAMISU_MFMA_NO_TAIL_SPLIT")) win_splits = (int)std::min<long>(std::min<long>(blocks, 2 * win_grid / rest), 16);
                if (win_splits < 2) win_splits = 1;
                // partial tiles of the pieces, a counter per remaining tile, the work queues' counters (pieces,
                // finished workgroups, one per XCD)
                const long cut = win_splits > 1 ? rest : 0;
                win_counters = cut + 2 + ttarget::XCDS;
                win_scratch_floats = cut * win_splits * BM * BN + win_counters;
            }
        }
    }

    // ---- kernel text
    c_printer dev;
    dev.fct = f;
    dev.device = true;
    std::set<std::string> used_buffers, used_scalars;
    dev.used_buffers = &used_buffers;
    dev.used_scalars = &used_scalars;
    std::set<std::string> locals = {"_accv", "_sum", "_r", "_c", "_x", "_k", "_u", "_cq"};
    for (int p : spatial) locals.insert(U.dims[p].kvar);
    for (int p : reduction) locals.insert(U.dims[p].kvar);
    if (batched) locals.insert(fuse->batch_iterator);

    // ---- the consumer's statements, once per point of the tile.  A value that the point itself stored
    // earlier is taken from its register instead of memory; a temporary of the function that nothing else
    // in the program reads is then not stored at all.
    std::ostringstream consumer_text, consumer_loads_text;
    std::set<std::string> dead;                 // buffers whose stores are dropped
    if (with_consumer) {
        struct stmt { const buffer *lhs; std::vector<expr> idx; std::string value, decl; primitive_t type; };
        std::vector<stmt> stmts;
        std::set<std::string> loaded;           // buffers that some statement still loads from memory
        std::map<std::string, std::pair<std::string, std::string>> latest;   // buffer -> (index text, value) of the point's latest store
        c_printer plain;
        plain.fct = f;
        plain.device = true;
        std::set<int> groups_used;
        std::vector<std::pair<std::string, expr>> hoisted;      // (variable, load) of what the points read from memory
        // an element as a text that is the same for every statement of a point: row and unit by their role,
        // outer dimensions by their value in terms of the host loops
        auto element_key = [&](size_t n, const buffer *b, const std::vector<expr> &index) {
            std::map<std::string, expr> m;
            for (size_t p = 0; p < xs[n].dims.size(); p++) {
                const canon_dim &d = xs[n].dims[p];
                if (!d.lo.is_defined()) continue;
                m[d.cvar] = (int)p == row_of[n] ? expr(var("_row")) : (int)p == unit_of[n] ? expr(var("_unit")) : xs[n].real->iterators.at(d.name);
            }
            std::vector<expr> v;
            for (auto &e : index) v.push_back(lir::simplify(e.substitute(m)));
            return b->get_name() + "[" + plain.print(lir::simplify(lir::linearize(b, v))) + "]";
        };
        // the element that statement w stores and the one statement n loads always differ by a non-zero
        // constant in some dimension (row and unit of the two points taken as unrelated)
        auto never_the_same = [&](size_t w, size_t n, const std::vector<expr> &loaded_index) {
            const std::vector<expr> &ia = xs[w].leaf->lhs_index;
            std::map<std::string, expr> ma, mb;
            for (auto &dd : xs[w].dims) if (dd.lo.is_defined()) ma[dd.cvar] = dd.in_kernel ? expr(var("_a_" + dd.cvar)) : xs[w].real->iterators.at(dd.name);
            for (auto &dd : xs[n].dims) if (dd.lo.is_defined()) mb[dd.cvar] = dd.in_kernel ? expr(var("_b_" + dd.cvar)) : xs[n].real->iterators.at(dd.name);
            for (size_t d = 0; d < ia.size() && d < loaded_index.size(); d++)
                if (differ_by_nonzero_constant(ia[d].substitute(ma), loaded_index[d].substitute(mb))) return true;
            return false;
        };
        for (size_t n = 0; n < xs.size(); n++) {
            canon &X = xs[n];
            bool okx = true;
            // on the canonical form: the result comes from the tile, a value the point stored earlier from its
            // register; any other load of a buffer that the consumer writes must be of an element that no
            // point of the launch stores
            expr val = X.leaf->rhs.transform([&](const expr &x) -> expr {
                if (!is_load(x)) return x;
                if (x.get_name() == acc_buf->get_name()) {
                    const int q = acc_group[n].at(x.to_str());
                    groups_used.insert(q);
                    return var(p_float32, "_g" + std::to_string(q));
                }
                const buffer *b = f->get_buffers().at(x.get_name());
                auto it = latest.find(x.get_name());
                const std::string key = element_key(n, b, x.get_access());
                if (it != latest.end() && it->second.first == key) return var(x.get_data_type(), it->second.second);
                for (size_t w = 0; w < xs.size(); w++) {
                    if (xs[w].leaf->lhs != b) continue;
                    if (element_key(w, b, xs[w].leaf->lhs_index) == key) continue;   // the point's own element, read from memory
                    if (!never_the_same(w, n, x.get_access())) okx = false;
                }
                loaded.insert(x.get_name());
                // what a point still reads from memory is read before any point of the thread stores (see below)
                const std::string name = "_in" + std::to_string(hoisted.size());
                hoisted.push_back({name, x.substitute(X.subs)});
                locals.insert(name);
                return var(x.get_data_type(), name);
            }).substitute(X.subs);
            if (!okx) return reject(36);
            stmt st;
            st.lhs = X.leaf->lhs;
            for (auto &e : X.leaf->lhs_index) st.idx.push_back(e.substitute(X.subs));
            st.value = "_v" + std::to_string(n);
            st.type = val.get_data_type();
            st.decl = "const " + primitive_c_name(st.type) + " " + st.value + " = " + dev.print(val) + ";";
            locals.insert(st.value);
            latest[st.lhs->get_name()] = {element_key(n, st.lhs, X.leaf->lhs_index), st.value};
            stmts.push_back(st);
        }
        // a temporary that only this kernel touches and never loads back from memory is not stored
        auto only_used_here = [&](const buffer *b) {
            if (b->get_argument_type() != a_temporary || !b->get_auto_allocate()) return false;
            for (auto *a : f->get_arguments()) if (a == b) return false;
            bool elsewhere = false;
            lir::walk(ctx.prog->root, [&](const node_ptr &x) {
                if (x->kind != node_kind::leaf) return;
                for (auto &l : leaves) if (l == x) return;
                for (auto &l : xleaves) if (l == x) return;
                if (x->lhs == b || x->copy_from == b || x->copy_to == b || x->target == b) { elsewhere = true; return; }
                for (const expr *e : {&x->rhs, &x->predicate})
                    if (e->is_defined() && reads_buffer(*e, b->get_name())) elsewhere = true;
                for (auto &l : x->lets) if (reads_buffer(l.second, b->get_name())) elsewhere = true;
                for (auto &ix : x->lhs_index) if (reads_buffer(ix, b->get_name())) elsewhere = true;
            });
            for (auto &inv : ctx.prog->invariants) if (reads_buffer(inv.value, b->get_name())) elsewhere = true;
            return !elsewhere;
        };
        for (auto &st : stmts)
            if (!loaded.count(st.lhs->get_name()) && only_used_here(st.lhs)) dead.insert(st.lhs->get_name());
        if (only_used_here(acc_buf)) dead.insert(acc_buf->get_name());
        const std::string m_var = U.dims[Mg[0]].kvar;
        // A thread handles _POINTS points.  Two passes: first everything the points read from memory (elements that
        // no point of the launch stores, or the point's own before it stores it), then values and stores.  Loads and
        // stores are counted by one in-order counter, so a point's load issued behind the previous point's stores
        // would wait for those stores to be acknowledged: a round trip to memory per point instead of one in all.
        std::ostringstream point;
        point << "        const int _p = threadIdx.x + _i * CFG::NT;\n";
        point << "        if (_p >= CFG::BM * " << UB << ") continue;\n";
        point << "        const int _lr = _p / " << UB << ", _lu = _p % " << UB << ";\n";
        if (edge) point << "        if (_tm * CFG::BM + _lr >= _M) continue;\n";
        point << "        const int32_t " << m_var << " = _tm * CFG::BM + _lr + (" << dev.print(U.dims[Mg[0]].lo.substitute(U.subs)) << ");\n";
        point << "        const int32_t _u = _tn * " << UB << " + _lu + (" << u_lo << ");\n";
        // (the loads do not depend on the contraction: they are issued before it and arrive while it runs)
        consumer_loads_text << "    constexpr int _POINTS = (CFG::BM * " << UB << " + CFG::NT - 1) / CFG::NT;\n";
        for (auto &hl : hoisted)
            consumer_loads_text << "    " << primitive_c_name(hl.second.get_data_type()) << " " << hl.first << "_of[_POINTS];\n";
        if (!hoisted.empty()) {
            consumer_loads_text << "#pragma unroll\n    for (int _i = 0; _i < _POINTS; _i++) {\n" << point.str();
            for (auto &hl : hoisted) consumer_loads_text << "        " << hl.first << "_of[_i] = " << dev.print(hl.second) << ";\n";
            consumer_loads_text << "    }\n";
        }
        consumer_text << "    __syncthreads();\n";
        consumer_text << "#pragma unroll\n    for (int _i = 0; _i < _POINTS; _i++) {\n" << point.str();
        for (auto &hl : hoisted)
            consumer_text << "        const " << primitive_c_name(hl.second.get_data_type()) << " " << hl.first << " = " << hl.first << "_of[_i];\n";
        for (int q : groups_used)
            consumer_text << "        const float _g" << q << " = _gt[_lr * (CFG::BN + 1) + " << q * UB << " + _lu];\n";
        for (auto &st : stmts) {
            consumer_text << "        " << st.decl << "\n";
            if (!dead.count(st.lhs->get_name())) consumer_text << "        " << dev.store(st.lhs, st.idx, st.value, st.type) << "\n";
        }
        consumer_text << "    }\n";
        for (int q = 0; q < G; q++) locals.insert("_g" + std::to_string(q));
    }
    auto replace_acc = [&](const expr &e) {
        return e.transform([&](const expr &x) -> expr {
            if (is_load(x) && x.get_name() == acc_buf->get_name()) return var(p_float32, "_accv");
            return x;
        });
    };
    // digits of a flattened index: "const int32_t _d<p> = lo + (flat / later extents) % extent;"
    auto digits = [&](const group_info &g, const std::string &flat, const std::string &ind, bool add_lo) {
        std::ostringstream os;
        if (g.dims.size() == 1) {
            os << ind << "const int32_t " << U.dims[g.dims[0]].kvar << " = " << flat;
            if (add_lo) os << " + (" << dev.print(U.dims[g.dims[0]].lo.substitute(U.subs)) << ")";
            os << ";\n";
            return os.str();
        }
        long later = 1;
        for (int q = (int)g.dims.size() - 1; q >= 0; q--) {
            os << ind << "const int32_t " << U.dims[g.dims[q]].kvar << " = ";
            if (q == 0) os << "(" << flat << " / " << later << ")";
            else os << "((" << flat << " / " << later << ") % " << g.ext[q] << ")";
            if (add_lo) os << " + (" << dev.print(U.dims[g.dims[q]].lo.substitute(U.subs)) << ")";
            os << ";\n";
            later *= g.ext[q];
        }
        return os.str();
    };
    std::ostringstream pre, body;
    const std::string cfg = "tgemm::config<" + std::to_string(BM) + ", " + std::to_string(BN) + ", " + std::to_string(BK) + ", " +
                            std::to_string(WGM) + ", " + std::to_string(WGN) + ", " + (operands[0].first.kmajor ? "true" : "false") + ", " +
                            (operands[0].second.kmajor ? "true" : "false") + ", " + (edge ? "true" : "false") + ", " + std::to_string(PADX) + ", " + std::to_string(WGK) + ", " + std::to_string(DEPTH) + ">";
    const int NT = 64 * WGM * WGN * WGK;
    if (bf16) {
        body << "    extern __shared__ __attribute__((aligned(16))) uint32_t _lds[];\n";
        // large tiles: slices go straight from global memory into a four-stage LDS ring
        if (BM >= 128) body << "    typedef tgemm::config_bf16_direct<" << BM << ", " << BN << ", " << BK << ", " << WGM << ", " << WGN << ", 4> CFG;\n";
        else body << "    typedef tgemm::config_bf16<" << BM << ", " << BN << ", " << BK << ", " << WGM << ", " << WGN << ", " << (edge ? "true" : "false") << "> CFG;\n";
    } else {
        body << "    extern __shared__ __attribute__((aligned(16))) float _lds[];\n";
        body << "    typedef " << cfg << " CFG;\n";
    }
    body << "    const int _M = " << dev.print(Me) << ", _N = " << dev.print(Ne) << ", _K = " << dev.print(Ke) << ";\n";
    body << "    int _tm, _tn;\n    tgemm::tile_of_block((_M + CFG::BM - 1) / CFG::BM, (_N + CFG::BN - 1) / CFG::BN, _tm, _tn);\n";
    body << "    tgemm::accumulators<CFG> _acc;\n    _acc.clear();\n" << consumer_loads_text.str();
    int term = 0, ktab_words = 0;
    const std::string kname = "_kernel_" + std::to_string(ctx.next_kernel_id());
    // several product terms over plain operands: one pipelined loop over the concatenated reduction ranges
    // (a call per term would drain and refill the pipeline between the terms)
    bool merge_terms = !bf16 && operands.size() > 1 && lit && Kl % 4 == 0 && !backend_option("TIRAMISU_MFMA_SEPARATE_TERMS");
    for (auto &o : operands) merge_terms = merge_terms && o.first.linear && o.second.linear;
    for (auto &o : operands) {
        if (!merge_terms || term == 0) body << "    {\n";
        if (bf16) {
            used_buffers.insert(o.first.buf->get_name());
            used_buffers.insert(o.second.buf->get_name());
            body << "        tgemm::tile_accumulate_bf16" << (BM >= 128 ? "_direct" : "") << "<CFG>(_acc, " << o.first.buf->get_name() << " + (" << dev.print(o.first.base) << "), "
                 << dev.print(o.first.ld) << ", " << o.second.buf->get_name() << " + (" << dev.print(o.second.base) << "), " << dev.print(o.second.ld)
                 << ", _M, _N, _K, _tm * CFG::BM, _tn * CFG::BN, _lds);\n    }\n";
            term++;
            continue;
        }
        if (windowed) {
            used_buffers.insert(o.first.buf->get_name());
            used_buffers.insert(o.second.buf->get_name());
            pre << "struct " << kname << "_taps {\n    static __device__ __forceinline__ constexpr int at(int t) {\n        return ";
            for (int t = 0; t + 1 < win_taps; t++) pre << "t == " << t << " ? " << win_tap_offsets[t] << " : ";
            pre << win_tap_offsets[win_taps - 1] << ";\n    }\n};\n";
            pre << "struct " << kname << "_pos {\n    __device__ __forceinline__ long operator()(int _x) const {\n" << digits(GN, "_x", "        ", false) << "        return 0";
            for (int p : GN.dims) pre << " + (long)" << U.dims[p].kvar << " * " << dev.print(o.second.coef.at(p));
            pre << ";\n    }\n};\n";
            std::ostringstream call;
            call << "    tgemm::contraction_window<CFG, " << win_cb << ", " << win_taps << ", " << win_floats << ", " << env_int("TIRAMISU_MFMA_WINDOW_AHEAD", 2) << ", " << win_splits << ", " << (env_int("TIRAMISU_MFMA_WINDOW_XCD_QUEUES", 1) ? "true" : "false") << ", " << kname << "_taps>("
                 << o.first.buf->get_name() << " + (" << dev.print(o.first.base) << "), " << dev.print(o.first.ld) << ", " << o.second.buf->get_name() << " + ("
                 << dev.print(o.second.base) << "), " << win_x_elements << "L, " << kname << "_pos(), " << win_chan_stride << "L, " << win_channels
                 << ", _M, _N, _tail_scratch, _lds, ";
            window_call_head = call.str();
            body << "    }\n";
            term++;
            continue;
        }
        int which = 0;
        for (const operand_info *g : {&o.first, &o.second}) {
            const std::string nm_text = std::string(which == 0 ? "_A" : "_B") + (merge_terms ? std::to_string(term) : "");
            const char *nm = nm_text.c_str();
            const group_info &rowg = which == 0 ? GM : GN;
            used_buffers.insert(g->buf->get_name());
            if (g->linear) {
                body << "        const float *" << nm << "p = " << g->buf->get_name() << " + (" << dev.print(g->base) << ");\n";
                body << "        const long " << nm << "ld = " << dev.print(g->ld) << ";\n";
                body << "        const tgemm::linear_source<" << (g->kmajor ? "true" : "false") << ", " << (edge ? "true" : "false") << "> " << nm
                     << "{" << nm << "p, " << nm << "ld, " << (which == 0 ? "_M" : "_N") << ", _K, (" << nm << "ld % 4 == 0) && ((uintptr_t)" << nm
                     << "p % 16 == 0)};\n";
            } else {
                // gather source: offsets are separable sums over the digits of the row and k indices
                const std::string sname = kname + "_src" + std::to_string(term) + (which == 0 ? "a" : "b");
                // 32-bit offsets when the buffer is small enough
                bool small = g->buf->has_constant_extents();
                if (small) {
                    double cnt = 1;
                    for (auto &d : g->buf->get_dim_sizes()) cnt *= (double)lir::simplify(d).get_int_val();
                    small = cnt < 2147483648.0;
                }
                const std::string OT = small ? "int32_t" : "long";
                // the k part of the offset (divisions by the extents of the reduction dimensions) is
                // tabulated in LDS once per workgroup when the table is small: one LDS read per load
                // instead of the digit arithmetic
                const bool tabulate = small && lit && Kl * 4 <= 32768 && ktab_words == 0 && !backend_option("TIRAMISU_MFMA_NO_KTAB");
                pre << "struct " << sname << " {\n    const float *__restrict__ base;\n    int XE, KE;\n    const int32_t *ktab;\n";
                pre << "    static __device__ __forceinline__ " << OT << " koff(int _k) {\n" << digits(GK, "_k", "        ", false) << "        return 0";
                for (int p : GK.dims) pre << " + (" << OT << ")" << U.dims[p].kvar << " * " << dev.print(g->coef.at(p));
                pre << ";\n    }\n";
                pre << "    __device__ __forceinline__ " << OT << " offset(int _x, int _k) const {\n";
                pre << digits(rowg, "_x", "        ", false);
                pre << "        return " << (tabulate ? "ktab[_k]" : "koff(_k)");
                for (int p : rowg.dims) pre << " + (" << OT << ")" << U.dims[p].kvar << " * " << dev.print(g->coef.at(p));
                pre << ";\n    }\n";
                if (tabulate) {
                    ktab_words = (int)((Kl + 3) / 4 * 4);
                    body << "        int32_t *_ktab = reinterpret_cast<int32_t *>(_lds) + CFG::LDS_BYTES / 4;\n";
                    body << "        for (int _k = threadIdx.x; _k < _K; _k += CFG::NT) _ktab[_k] = " << sname << "::koff(_k);\n";
                    body << "        __syncthreads();\n";
                }
                pre << "    __device__ __forceinline__ tgemm::f32x4 load4(int x, int k) const {\n";
                const char *full = g->gather_kdir ? "(x < XE && k + 3 < KE)" : "(k < KE && x + 3 < XE)";
                if (g->gather_vec)
                    pre << "        if (" << (edge ? full : "true") << ") { tgemm::f32x4_u v = *reinterpret_cast<const tgemm::f32x4_u *>(base + offset(x, k)); "
                           "return tgemm::f32x4{v[0], v[1], v[2], v[3]}; }\n";
                pre << "        tgemm::f32x4 r = {0.f, 0.f, 0.f, 0.f};\n";
                pre << "        for (int e = 0; e < 4; e++) {\n            const int xx = " << (g->kmajor ? "x" : "x + e") << ", kk = " << (g->kmajor ? "k + e" : "k")
                    << ";\n            if (xx < XE && kk < KE) r[e] = base[offset(xx, kk)];\n        }\n        return r;\n    }\n};\n";
                body << "        const " << sname << " " << nm << "{" << g->buf->get_name() << " + (" << dev.print(g->base) << "), " << (which == 0 ? "_M" : "_N")
                     << ", _K, " << (tabulate ? "_ktab" : "nullptr") << "};\n";
            }
            which++;
        }
        term++;
        if (merge_terms && term < (int)operands.size()) continue;
        std::string a_name = "_A", b_name = "_B", k_text = "_K";
        if (merge_terms) {
            a_name = "_A0";
            b_name = "_B0";
            for (int t = 1; t < term; t++) {
                for (std::string *nm : {&a_name, &b_name}) {
                    const std::string next = std::string(nm == &a_name ? "_A" : "_B") + std::to_string(t), cat = *nm + "c";
                    body << "        const tgemm::concat_k<decltype(" << *nm << "), decltype(" << next << ")> " << cat << "{" << *nm << ", " << next << ", " << t << " * _K};\n";
                    *nm = cat;
                }
            }
            k_text = std::to_string(term) + " * _K";
        }
        if (with_consumer) {
            body << "        const tgemm::regrouped_rows<decltype(" << b_name << "), CFG::BN, " << UB << "> _Bq{" << b_name << ", " << UE << "};\n";
            b_name = "_Bq";
        }
        body << "        tgemm::tile_accumulate<CFG>(_acc, " << a_name << ", " << b_name << ", " << k_text << ", _tm * CFG::BM, _tn * CFG::BN, _lds);\n    }\n";
    }
    if (with_consumer)   // the finished tile, handed to the consumer's statements through LDS (behind the operand stages)
        body << "    float *_gt = _lds + CFG::LDS_BYTES / 4 + " << ktab_words << ";\n";
    // The element-wise tail of a tile: `_accv` = initial value + sum, then the store of the accumulator element and/or of the
    // fused epilogue's value.  With a single store the tail is printed as two functions, value and store, and
    // tile_epilogue runs the first over the whole tile before the second: loads and stores are counted by one in-order
    // counter, so a load behind a store can only be waited for together with that store's acknowledgement, and
    // element-by-element the tile would pay one round trip to memory per element.
    std::string digit_text;
    if (with_consumer) {
        digit_text = digits(GM, "_r", "        ", true);
        digit_text += "        const int _cq = tgemm::regrouped_index<CFG::BN, " + std::to_string(UB) + ">(_c, " + std::to_string(UE) + ");\n";
        digit_text += digits(GN, "_cq", "        ", true);
    } else {
        digit_text = digits(GM, "_r", "        ", true) + digits(GN, "_c", "        ", true);
    }
    std::vector<expr> acc_index;
    for (auto &e : U.leaf->lhs_index) acc_index.push_back(e.substitute(U.subs));
    std::string accv_text;
    if (has_init) {
        expr init = cs[ii].leaf->rhs.substitute(cs[ii].subs);
        expr z = lir::simplify(init);
        if (z.is_constant() && z.get_double_val() == 0.0) accv_text = "        float _accv = _sum;\n";
        else accv_text = "        float _accv = " + dev.print(init) + " + _sum;\n";
    } else {
        accv_text = "        float _accv = " + dev.element(acc_buf, acc_index) + " + _sum;\n";
    }
    if (with_consumer) accv_text += "        _gt[(_r - _tm * CFG::BM) * (CFG::BN + 1) + (_c - _tn * CFG::BN)] = _accv;\n";
    const bool acc_stored = !acc_private && !dead.count(acc_buf->get_name()) &&
        !(has_epi && cs[ei].leaf->lhs == acc_buf && same_element(expr(o_access, acc_buf->get_name(), leaves[ei]->lhs_index, p_float32), acc_buf, ureal->lhs_index));
    std::string epi_value_text, epi_store_text, epi_one_pass_text;   // of the fused epilogue: its value (reads _accv), its store of `_v`, both in one
    bool epi_is_float = true;
    if (has_epi) {
        canon &E = cs[ei];
        std::vector<expr> ix;
        for (auto &e : E.leaf->lhs_index) ix.push_back(e.substitute(E.subs));
        expr val = replace_acc(E.leaf->rhs.substitute(E.subs));
        epi_is_float = val.get_data_type() == p_float32;
        epi_value_text = dev.print(val);
        epi_store_text = dev.store(E.leaf->lhs, ix, "_v", val.get_data_type());
        epi_one_pass_text = dev.store(E.leaf->lhs, ix, epi_value_text, val.get_data_type());
    }
    const bool two_pass = !(acc_stored && has_epi) && epi_is_float && !backend_option("TIRAMISU_MFMA_ONE_PASS_EPILOGUE");
    if (two_pass) {
        body << "    auto _epi_value = [&](int _r, int _c, float _sum) -> float {\n" << digit_text << accv_text;
        body << "        return " << (has_epi ? epi_value_text : std::string("_accv")) << ";\n    };\n";
        body << "    auto _epi_store = [&](int _r, int _c, float _v) {\n" << digit_text;
        if (has_epi) body << "        " << epi_store_text << "\n";
        else if (acc_stored) body << "        " << dev.store(acc_buf, acc_index, "_v", p_float32) << "\n";
        body << "    };\n";
    } else {
        body << "    auto _epi = [&](int _r, int _c, float _sum) {\n" << digit_text << accv_text;
        if (acc_stored) body << "        " << dev.store(acc_buf, acc_index, "_accv", p_float32) << "\n";
        if (has_epi) body << "        " << epi_one_pass_text << "\n";
        body << "    };\n";
    }
    const std::string epi_args = two_pass ? "_epi_value, _epi_store" : "_epi";
    if (windowed) {
        body << window_call_head << epi_args << ");\n";
    } else {
        if (WGK > 1) body << "    if (tgemm::tile_reduce_k<CFG>(_acc, _lds))\n    ";
        body << "    tgemm::tile_epilogue<CFG>(_acc, _M, _N, _tm * CFG::BM, _tn * CFG::BN, " << epi_args << ");\n";
    }
    body << consumer_text.str();

    kernel k;
    k.name = kname;
    bool any_gather = false;
    for (auto &o : operands) any_gather = any_gather || !o.first.linear || !o.second.linear;
    k.how = std::string("mfma-contraction: ") + (bf16 ? (BM >= 128 ? "v_mfma_f32_32x32x16_bf16, slices loaded straight into LDS, " : "v_mfma_f32_32x32x16_bf16, ") : "v_mfma_f32_32x32x2_f32, ") + (windowed ? "implicit GEMM, sliding window of " + std::to_string(win_taps) + " taps staged in LDS by blocks of " + std::to_string(win_cb) + " channels, " :
                                                                                      any_gather ? "implicit GEMM (gathered operand), " : "") + "M " +
            std::to_string(Mg.size()) + " dim(s) x N " + std::to_string(Ng.size()) + " x K " + std::to_string(Kg.size()) + ", tile " +
            std::to_string(BM) + "x" + std::to_string(BN) + "x" + std::to_string(BK) + (edge ? ", guarded edges" : ", whole tiles") + ", " +
            std::to_string(operands.size()) + " product term(s)" + (has_init ? ", fused initialisation" : "") + (has_epi ? ", fused epilogue" : "") +
            (with_consumer ? ", " + std::to_string(xs.size()) + " point-wise statement(s) of the following nest fused (" + std::to_string(G) + " column group(s) per unit, " +
                                 std::to_string(dead.size()) + " temporaries kept in registers)" : "") +
            (batched ? ", iterations of the parallel host loop as gridDim.z" : "") +
            (windowed ? ", " + std::to_string(win_resident) + " workgroup(s) per compute unit take tiles from a queue" + (win_splits > 1 ? ", the last tiles cut into " + std::to_string(win_splits) + " pieces" : std::string()) : std::string());
    std::ostringstream host;
    host << "    {\n";
    // With a batched launch the values of the outer dimensions depend on blockIdx.z: they are computed
    // in the kernel from the iterators of the enclosing host loops, which become its parameters.
    std::ostringstream batch_prologue;
    if (batched) {
        batch_prologue << "    const int32_t " << fuse->batch_iterator << " = (int32_t)blockIdx.z + _batch_first;\n";
        std::set<std::string> declared;
        for (auto &o : outers)
            if (used_scalars.count(o.name) && declared.insert(o.name).second) {
                batch_prologue << "    const int32_t " << o.name << " = " << dev.print(o.host_value) << ";\n";
                locals.insert(o.name);
            }
        used_scalars.insert("_batch_first");
    }
    for (auto &nm : used_scalars) {
        if (locals.count(nm)) continue;
        primitive_t t = p_int32;
        bool known = nm == "_batch_first";
        for (auto &o : outers)
            if (o.name == nm) known = true;
        for (auto c : f->get_invariants())
            if (c->get_name() == nm) { t = c->get_data_type(); known = true; }
        for (auto &it : ctx.host_iterators)
            if (batched && it == nm) known = true;
        if (!known) return reject(21);
        k.params.push_back({false, nm, t});
    }
    {
        c_printer hp;
        hp.fct = f;
        std::set<std::string> declared;
        if (batched) {
            host << "        const int32_t _batch_first = " << hp.print(fuse->batch_first) << ";\n";
            k.grid[2] = "((" + hp.print(fuse->batch_last) + ") >= _batch_first ? (" + hp.print(fuse->batch_last) + ") - _batch_first + 1 : 0)";
        }
        for (auto &o : outers)
            if (!batched && used_scalars.count(o.name) && declared.insert(o.name).second)
                host << "        const int32_t " << o.name << " = " << hp.print(o.host_value) << ";\n";
        // grid: number of tiles (outer parameters are in scope here)
        k.grid[0] = "((" + hp.print(Me) + " + " + std::to_string(BM - 1) + ") / " + std::to_string(BM) + ") * ((" + hp.print(Ne) + " + " +
                    std::to_string(BN - 1) + ") / " + std::to_string(BN) + ")";
    }
    for (auto &nm : used_buffers) {
        buffer *b = f->get_buffers().at(nm);
        if (b->get_location() != memory_location::global) return reject(22);
        k.params.push_back({true, nm, b->get_elements_type()});
    }
    if (windowed) {
        // scratch for the pieces of the last round's tiles and their counters: kept by the runtime, one block per host
        // thread and stream (a call works on the thread's current stream; calls of one thread on two streams may overlap
        // and must not share queues and counters), allocated at the first call there; the counters start at zero and
        // every launch leaves them at zero
        // (buffer parameters stay sorted by name)
        auto at = k.params.begin();
        while (at != k.params.end() && (!at->is_buffer || at->name < "_tail_scratch")) ++at;
        k.params.insert(at, {true, "_tail_scratch", p_float32});
        k.grid[0] = std::to_string(win_grid);
        host << "        static const char _tail_site = 0;\n";
        host << "        int32_t _tail_fresh = 0;\n";
        host << "        float *_tail_scratch = (float *)tiramisu_hip_kept_scratch(&_tail_site, (uint64_t)" << win_scratch_floats << " * sizeof(float), &_tail_fresh);\n";
        host << "        if (_tail_fresh) {\n";
        host << "            static const uint32_t _zeros[" << win_counters << "] = {};\n";
        host << "            tiramisu_hip_memcpy_to_device((void *)(_tail_scratch + " << (win_scratch_floats - win_counters) << "), (void *)_zeros, sizeof(_zeros));\n";
        host << "        }\n";
    }
    k.block[0] = std::to_string(NT);
    // two LDS stages of an A and a B slice
    {
        const int rowA = operands[0].first.kmajor ? (BK / 4) * (BM + PADX) * 4 : BK * BM;
        const int rowB = operands[0].second.kmajor ? (BK / 4) * (BN + PADX) * 4 : BK * BN;
        k.lds_bytes = std::to_string(2 * (rowA + rowB) * 4);
        if (bf16) k.lds_bytes = std::to_string((BM >= 128 ? 4 : 2) * (BK / 8) * (BM + BN) * 4 * 4);   // four-stage ring for the large tiles
        else if (ktab_words) k.lds_bytes = std::to_string(2 * (rowA + rowB) * 4 + ktab_words * 4);
        if (with_consumer) k.lds_bytes = std::to_string(std::stol(k.lds_bytes) + BM * (BN + 1) * 4);
        if (windowed) k.lds_bytes = std::to_string(2 * ((long)win_cb * (win_taps * BM + 32) + (long)win_cb * win_floats) * 4);
    }
    std::ostringstream src;
    src << pre.str();
    src << "extern \"C\" __global__ void __launch_bounds__(" << NT;
    if (windowed && win_resident > 1) src << ", " << win_resident * (NT / 64) / 4;       // waves per SIMD: bounds the registers
    src << ") " << k.name << "(";
    for (size_t i = 0; i < k.params.size(); i++) {
        auto &p = k.params[i];
        src << (i ? ", " : "");
        if (p.is_buffer) src << primitive_c_name(p.type) << " *__restrict__ " << p.name;
        else src << "const " << primitive_c_name(p.type) << " " << p.name;
    }
    src << ")\n{\n" << batch_prologue.str() << body.str() << "}\n";
    k.source = src.str();
    add_include_once(ctx, "#include \"gemm_mfma.hip.h\"");
    if (bf16) add_include_once(ctx, "#include \"gemm_mfma_bf16.hip.h\"");
    if (windowed) add_include_once(ctx, "#include \"gemm_mfma_window.hip.h\"");
    host << launch_text(k, "        ") << "    }\n";
    plan.kernels.push_back(k);
    plan.host_code = host.str();
    return true;
}

}  // namespace hipgen
}  // namespace tiramisu
