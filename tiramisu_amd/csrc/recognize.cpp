// Pattern-directed kernel emitters.  A GPU-mapped loop nest is handed to these before the
// schedule-faithful emitter; each one checks -- on the computations' expressions, iteration
// domains and store relations, with isl where sets and maps are compared -- that the nest is of
// its kind, and only then replaces it by kernels shaped for gfx950.  Anything that fails a check
// falls back to the generic emitter, which reproduces the reference's behaviour.
#include <cstdlib>
#include <sstream>

#include "hip_backend.h"
#include "isl_api.h"
#include "util.h"

namespace tiramisu {
namespace hipgen {

using lir::leaf_kind;
using lir::node;
using lir::node_kind;
using lir::node_ptr;

namespace {

#ifndef TIRAMISU_AMD_KERNEL_DIR
#define TIRAMISU_AMD_KERNEL_DIR "."
#endif

std::string kernel_dir() {
    if (const char *e = std::getenv("TIRAMISU_AMD_KERNEL_DIR")) return e;
    return TIRAMISU_AMD_KERNEL_DIR;
}

int env_int(const char *name, int dflt) {
    const char *e = std::getenv(name);
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

void leaves_under(const node_ptr &n, std::vector<node_ptr> &out, bool &has_cond) {
    lir::walk(n, [&](const node_ptr &x) {
        if (x->kind == node_kind::leaf) out.push_back(x);
        if (x->kind == node_kind::cond) has_cond = true;
    });
}

void add_include_once(context &ctx, const std::string &line) {
    if (ctx.include_once.insert(line).second) ctx.includes += line + "\n";
}

}  // namespace

// ------------------------------------------------------------------------------------------
// Stencil over a ping-pong pair of planes inside a host time loop:
//     S(t, y, x) = f( S(t-1, y+dy, x+dx) ... ),   S stored at B[t mod 2, y, x].
// Every read at step t is of step t-1 within a constant radius, so all flow dependences have
// distance (1, dy, dx) and overlapped time tiles are legal; the time loop is replaced by
// launches that each advance an odd number of steps (see kernels/stencil2d.hip.h).
bool emit_stencil(context &ctx, const node_ptr &root, const node_ptr &time_loop, launch_plan &plan) {
    // either a host time loop around a mapped nest, or a mapped nest whose time step is fixed
    // (a one-step time loop has no loop node in the AST)
    if ((!time_loop && !root) || (time_loop && root)) return false;
    if (std::getenv("TIRAMISU_NO_STENCIL")) return false;
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
    if (its.size() != 3 || S->get_data_type() != p_float32) return false;
    auto t_it = leaf->iterators.find(its[0]);
    if (t_it == leaf->iterators.end()) return false;
    if (time_loop) {
        if (t_it->second.get_expr_type() != e_var || t_it->second.get_name() != time_loop->iterator) return false;
    } else if (!lir::simplify(t_it->second).is_integer_literal()) {
        return false;
    }

    // expression: reads of S at (t-1, y+dy, x+dx) and float literals only
    int radius = 0;
    bool ok = true;
    std::function<expr(const expr &)> rewrite = [&](const expr &e) -> expr {
        if (!e.is_defined()) { ok = false; return e; }
        switch (e.get_expr_type()) {
        case e_val: return e;
        case e_op: {
            if (e.get_op_type() == o_access) {
                long dt, dy, dx;
                if (e.get_name() != S->get_name() || e.get_access().size() != 3 || !var_plus_const(e.get_access()[0], its[0], dt) ||
                    !var_plus_const(e.get_access()[1], its[1], dy) || !var_plus_const(e.get_access()[2], its[2], dx) || dt != -1) {
                    ok = false;
                    return e;
                }
                radius = std::max<long>(radius, std::max(std::labs(dy), std::labs(dx)));
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
    if (!ok || radius < 1 || radius > 4) return false;

    // store relation and buffer
    buffer *B = leaf->lhs;
    if (!B || B->get_location() != memory_location::global || B->get_n_dims() != 3 || !B->has_constant_extents()) return false;
    if (lir::simplify(B->get_dim_sizes()[0]).get_int_val() != 2) return false;
    const long NY = lir::simplify(B->get_dim_sizes()[1]).get_int_val(), NX = lir::simplify(B->get_dim_sizes()[2]).get_int_val();
    if (!access_equals(S, "{ " + S->get_name() + "[t,y,x] -> " + B->get_name() + "[t mod 2, y, x] }")) return false;

    // iteration domain: a box that keeps the stencil inside the plane
    std::vector<long> lo, hi;
    if (!literal_box(S, lo, hi)) return false;
    if (lo[1] - radius < 0 || hi[1] + radius > NY - 1 || lo[2] - radius < 0 || hi[2] + radius > NX - 1) return false;

    // ---- plan: odd chunks for all steps but the last, then the last step alone, so that on
    // return both planes hold exactly what the un-tiled loop leaves there
    const long T0 = lo[0], T1 = hi[0];
    const long steps = T1 - T0 + 1;
    int rmax = env_int("TIRAMISU_STENCIL_STEPS", 5);
    if (rmax % 2 == 0) rmax -= 1;
    if (rmax < 1) rmax = 1;
    const int TW = env_int("TIRAMISU_STENCIL_TW", 256), TH = env_int("TIRAMISU_STENCIL_TH", 32);
    const int NT = env_int("TIRAMISU_STENCIL_THREADS", 512);
    std::vector<std::pair<long, int>> chunks;  // (first step, number of steps)
    long t = T0, rem = steps - 1;
    while (rem > 0) {
        int c = (int)std::min<long>(rmax, rem);
        if (c % 2 == 0) c -= 1;
        chunks.push_back({t, c});
        t += c;
        rem -= c;
    }
    chunks.push_back({t, 1});

    c_printer dev;
    dev.fct = f;
    dev.device = true;
    const std::string point_text = dev.print(point);
    std::map<int, kernel> by_steps;
    std::ostringstream host;
    for (auto &ch : chunks) {
        if (!by_steps.count(ch.second)) {
            kernel k;
            k.name = "_kernel_" + std::to_string(ctx.next_kernel_id());
            k.how = "stencil: " + std::to_string(ch.second) + " time step(s) per launch, radius " + std::to_string(radius) +
                    ", tile " + std::to_string(TH) + "x" + std::to_string(TW) + ", LDS halo";
            std::ostringstream s;
            s << "#define ST_NAME " << k.name << "\n#define ST_NY " << NY << "\n#define ST_NX " << NX << "\n#define ST_Y0 " << lo[1]
              << "\n#define ST_Y1 " << hi[1] << "\n#define ST_X0 " << lo[2] << "\n#define ST_X1 " << hi[2] << "\n#define ST_TH " << TH
              << "\n#define ST_TW " << TW << "\n#define ST_R " << ch.second << "\n#define ST_RAD " << radius << "\n#define ST_NT " << NT
              << "\n#define ST_EXPR " << point_text << "\n#include \"" << kernel_dir() << "/stencil2d.hip.h\"\n"
              << "#undef ST_NAME\n#undef ST_NY\n#undef ST_NX\n#undef ST_Y0\n#undef ST_Y1\n#undef ST_X0\n#undef ST_X1\n#undef ST_TH\n"
              << "#undef ST_TW\n#undef ST_R\n#undef ST_RAD\n#undef ST_NT\n#undef ST_EXPR\n";
            k.source = s.str();
            k.params = {{true, B->get_name(), B->get_elements_type()}, {false, "_st_src", p_int32}};
            k.grid[0] = std::to_string((NX + TW - 1) / TW);
            k.grid[1] = std::to_string((NY + TH - 1) / TH);
            k.block[0] = std::to_string(NT);
            by_steps[ch.second] = k;
        }
        const long src = (((ch.first - 1) % 2) + 2) % 2;
        host << "    {\n        const int32_t _st_src = " << src << ";  // steps " << ch.first << ".." << ch.first + ch.second - 1 << "\n"
             << launch_text(by_steps[ch.second], "        ") << "    }\n";
    }
    for (auto &kv : by_steps) plan.kernels.push_back(kv.second);
    plan.host_code = host.str();
    return true;
}

bool emit_contraction(context &, const node_ptr &, launch_plan &) { return false; }

}  // namespace hipgen
}  // namespace tiramisu
