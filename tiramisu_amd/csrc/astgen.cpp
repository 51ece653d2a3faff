// From schedules to the lowered loop program: builds the isl AST of a function
// (same build options as the reference, src/tiramisu_function.cpp:1375-1456), and at every
// statement instance turns the computation into a leaf whose buffer indices are expressions
// of the AST loop iterators.  Accesses are lowered by composing, in isl, the inverse of the
// statement's schedule inside the current build with the accessed computation's store
// relation, and asking the build for the index expressions -- so that "i % 16" with
// i = 16*c1 + c3 comes out as "c3" (the reference reaches the same result through
// tiramisu_codegen_halide.cpp:1292-1440 and :3339-3440).
#include <tiramisu/core.h>

#include <algorithm>
#include <cstdint>
#include <sstream>

#include <tiramisu/isl_api.h>
#include "lir.h"
#include "util.h"

namespace tiramisu {

using lir::node;
using lir::node_kind;
using lir::node_ptr;
using lir::leaf_kind;

namespace {

struct lowering {
    function *f;
    std::vector<node_ptr> leaves;
    int placeholder_counter = 0;
    bool as_written = false;   // lower expressions as they were before cache_shared() redirected loads

    primitive_t scalar_type(const std::string &nm) const {
        for (auto c : f->get_invariants())
            if (c->get_name() == nm) return c->get_data_type();
        return global::get_loop_iterator_data_type();
    }

    expr from_isl(isl_ast_expr *e, const std::map<std::string, expr> &subs) {
        expr r;
        switch (isl_ast_expr_get_type(e)) {
        case isl_ast_expr_id: {
            isl_id *id = isl_ast_expr_get_id(e);
            std::string nm = isl_id_get_name(id);
            isl_id_free(id);
            auto it = subs.find(nm);
            r = (it != subs.end()) ? it->second : expr(var(scalar_type(nm), nm));
            break;
        }
        case isl_ast_expr_int: {
            isl_val *v = isl_ast_expr_get_val(e);
            r = value_cast(global::get_loop_iterator_data_type(), (int64_t)isl_val_get_num_si(v));
            isl_val_free(v);
            break;
        }
        case isl_ast_expr_op: {
            int n = isl_ast_expr_get_op_n_arg(e);
            std::vector<expr> a;
            isl_ast_op_type ot = isl_ast_expr_get_op_type(e);
            for (int i = (ot == isl_ast_op_access || ot == isl_ast_op_call) ? 1 : 0; i < n; i++) {
                isl_ast_expr *s = isl_ast_expr_get_op_arg(e, i);
                a.push_back(from_isl(s, subs));
                isl_ast_expr_free(s);
            }
            auto fold = [&](op_t o) {
                expr acc = expr(o, a[0], a[1]);
                for (size_t i = 2; i < a.size(); i++) acc = expr(o, acc, a[i]);
                return acc;
            };
            switch (ot) {
            case isl_ast_op_and: case isl_ast_op_and_then: r = fold(o_logical_and); break;
            case isl_ast_op_or: case isl_ast_op_or_else: r = fold(o_logical_or); break;
            case isl_ast_op_max: r = fold(o_max); break;
            case isl_ast_op_min: r = fold(o_min); break;
            case isl_ast_op_minus: r = expr(o_minus, a[0]); break;
            case isl_ast_op_add: r = expr(o_add, a[0], a[1]); break;
            case isl_ast_op_sub: r = expr(o_sub, a[0], a[1]); break;
            case isl_ast_op_mul: r = expr(o_mul, a[0], a[1]); break;
            case isl_ast_op_div: r = expr(o_div, a[0], a[1]); break;        // exact
            case isl_ast_op_fdiv_q: r = expr(o_floordiv, a[0], a[1]); break;
            case isl_ast_op_pdiv_q: r = expr(o_div, a[0], a[1]); break;     // dividend >= 0
            case isl_ast_op_pdiv_r: r = expr(o_mod, a[0], a[1]); break;     // dividend >= 0
            case isl_ast_op_zdiv_r: r = expr(o_mod, a[0], a[1]); break;     // only compared with 0
            case isl_ast_op_cond: case isl_ast_op_select: r = expr(o_select, a[0], a[1], a[2]); break;
            case isl_ast_op_eq: r = expr(o_eq, a[0], a[1]); break;
            case isl_ast_op_le: r = expr(o_le, a[0], a[1]); break;
            case isl_ast_op_lt: r = expr(o_lt, a[0], a[1]); break;
            case isl_ast_op_ge: r = expr(o_ge, a[0], a[1]); break;
            case isl_ast_op_gt: r = expr(o_gt, a[0], a[1]); break;
            case isl_ast_op_access: {
                isl_ast_expr *b = isl_ast_expr_get_op_arg(e, 0);
                isl_id *id = isl_ast_expr_get_id(b);
                std::string bn = isl_id_get_name(id);
                isl_id_free(id);
                isl_ast_expr_free(b);
                auto it = f->get_buffers().find(bn);
                if (it == f->get_buffers().end()) ERROR("access to unknown buffer " + bn, true);
                r = expr(o_access, bn, a, it->second->get_elements_type());
                break;
            }
            default: ERROR("unsupported isl AST operator", true);
            }
            break;
        }
        default: ERROR("unsupported isl AST expression", true);
        }
        return lir::simplify(r);
    }

    computation *find_computation(const std::string &nm) const {
        auto v = f->get_computation_by_name(nm);
        for (auto c : f->get_invariants())
            if (c->get_name() == nm) return c;
        return v.empty() ? nullptr : v[0];
    }

    // Index expressions of the buffer element that computation X stores its instance
    // X(args) in, seen from a statement instance of L inside `build`.
    expr lower_access(isl_ast_build *build, computation *L, const std::map<std::string, expr> &iters,
                      computation *X, const std::vector<expr> &args) {
        if (!X->get_access_relation())
            ERROR("computation " + X->get_name() + " is accessed but not mapped to a buffer (store_in)", true);
        std::vector<std::string> params = f->get_invariant_names();
        std::map<std::string, expr> subs;
        std::vector<std::string> arg_strs;
        for (auto &a : args) {
            bool ok = true;
            std::string s = expr_to_isl_str(a, ok);
            if (ok) {
                // every variable must be an iterator of L or an invariant
                a.visit([&](const expr &x) {
                    if (x.get_expr_type() == e_var && !iters.count(x.get_name()) &&
                        std::find(params.begin(), params.end(), x.get_name()) == params.end())
                        ok = false;
                });
            }
            if (!ok) {
                std::string ph = "_na" + std::to_string(placeholder_counter++);
                subs[ph] = lower_expr(build, L, iters, a);
                params.push_back(ph);
                s = ph;
            }
            arg_strs.push_back(s);
        }
        if (args.empty()) arg_strs.push_back("0");
        std::string ms = (params.empty() ? std::string() : "[" + join(params, ", ") + "] -> ") + "{ " + L->get_name() +
                         "[" + join(L->get_iteration_domain_dimension_names(), ", ") + "] -> " + X->get_name() + "[" +
                         join(arg_strs, ", ") + "] }";
        isl_map *arg_map = isl_map_read_from_str(f->get_isl_ctx(), ms.c_str());
        if (!arg_map) ERROR("cannot build access map " + ms, true);
        isl_map *to_buf = isl_map_apply_range(arg_map, isl_map_copy(X->get_access_relation()));
        isl_map *sched = isl_map_from_union_map(isl_ast_build_get_schedule(build));
        isl_map *full = isl_map_apply_range(isl_map_reverse(sched), to_buf);
        isl_pw_multi_aff *pma = isl_pw_multi_aff_from_map(full);
        if (!pma) ERROR("access of " + L->get_name() + " to " + X->get_name() + " is not a function of the loop iterators", true);
        isl_ast_expr *ae = isl_ast_build_access_from_pw_multi_aff(build, pma);
        if (!ae) ERROR("isl could not build the access expression " + ms, true);
        expr r = from_isl(ae, subs);
        isl_ast_expr_free(ae);
        return r;
    }

    expr lower_expr(isl_ast_build *build, computation *L, const std::map<std::string, expr> &iters, const expr &e) {
        if (!e.is_defined()) return e;
        switch (e.get_expr_type()) {
        case e_val: case e_sync: return e;
        case e_var: {
            auto it = iters.find(e.get_name());
            return it != iters.end() ? it->second : e;
        }
        case e_op: {
            if (e.get_op_type() == o_access) {
                computation *X = find_computation(e.get_name());
                if (X && X->is_let_stmt()) return var(X->get_data_type(), X->get_name());
                if (X) return lower_access(build, L, iters, X, e.get_access());
                if (f->get_buffers().count(e.get_name())) {  // already names a buffer
                    std::vector<expr> idx;
                    for (auto &a : e.get_access()) idx.push_back(lower_expr(build, L, iters, a));
                    return expr(o_access, e.get_name(), idx, e.get_data_type());
                }
                ERROR("access to undeclared computation " + e.get_name(), true);
            }
            if (e.get_op_type() == o_address) {
                // expr(o_address, var("S0")): the halide_buffer_t of the buffer that computation S0 is stored in, for
                // an external function (reference: tiramisu_codegen_halide.cpp:3830-3835, "<buffer>.buffer")
                const std::string &nm = e.get_operand(0).get_name();
                computation *X = find_computation(nm);
                const buffer *b = X ? X->get_buffer() : (f->get_buffers().count(nm) ? f->get_buffers().at(nm) : nullptr);
                if (!b) ERROR("address of " + nm + ": neither a computation with a buffer nor a buffer", true);
                return expr(o_address, expr(o_buffer, b->get_name()));
            }
            expr r = e;
            std::vector<expr> ops, args;
            for (auto &o : e.get_operands()) ops.push_back(lower_expr(build, L, iters, o));
            for (auto &a : e.get_arguments()) args.push_back(lower_expr(build, L, iters, a));
            switch (e.get_n_arg()) {
            case 1:
                r = (e.get_op_type() == o_cast) ? expr(o_cast, e.get_data_type(), ops[0]) : expr(e.get_op_type(), ops[0]);
                break;
            case 2: r = expr(e.get_op_type(), ops[0], ops[1]).copy_with_type(e.get_data_type()); break;
            case 3: r = expr(e.get_op_type(), ops[0], ops[1], ops[2]); break;
            default: r = expr(e.get_op_type(), e.get_name(), args, e.get_data_type()); break;
            }
            return r;
        }
        default: return e;
        }
    }

    node_ptr make_leaf(isl_ast_build *build, computation *C, isl_ast_expr *call) {
        node_ptr n = std::make_shared<node>();
        n->kind = node_kind::leaf;
        n->comp = C;
        int na = isl_ast_expr_get_op_n_arg(call);
        const auto &names = C->get_iteration_domain_dimension_names();
        for (int i = 1; i < na && i - 1 < (int)names.size(); i++) {
            isl_ast_expr *a = isl_ast_expr_get_op_arg(call, i);
            n->iterators[names[i - 1]] = from_isl(a, {});
            isl_ast_expr_free(a);
        }
        const expr &e = (as_written && C->get_uncached_expr().is_defined()) ? C->get_uncached_expr() : C->get_expr();
        auto find_buffer = [&](const std::string &bn) {
            auto it = f->get_buffers().find(bn);
            if (it == f->get_buffers().end()) ERROR("unknown buffer " + bn + " in " + C->get_name(), true);
            return it->second;
        };
        if (e.get_expr_type() == e_sync) {
            n->lkind = leaf_kind::sync;
            return n;
        }
        if (e.get_expr_type() == e_op && e.get_op_type() == o_memcpy) {
            n->lkind = leaf_kind::copy;
            n->copy_from = find_buffer(e.get_operand(0).get_name());
            n->copy_to = find_buffer(e.get_operand(1).get_name());
            return n;
        }
        if (e.get_expr_type() == e_op && (e.get_op_type() == o_allocate || e.get_op_type() == o_free)) {
            n->lkind = e.get_op_type() == o_allocate ? leaf_kind::allocate : leaf_kind::release;
            n->target = find_buffer(e.get_name());
            return n;
        }
        if (!e.is_defined()) ERROR("computation " + C->get_name() + " is scheduled but has no expression", true);
        n->lkind = (e.get_expr_type() == e_op && e.get_op_type() == o_call) ? leaf_kind::call : leaf_kind::assign;
        // a scheduled constant declares a scalar visible to what follows it in its loop body
        // (reference: tiramisu_codegen_cuda.cpp:658-676)
        if (C->is_let_stmt()) n->lkind = leaf_kind::let;
        for (auto &l : C->get_associated_let_stmts())
            n->lets.push_back({l.first, lower_expr(build, C, n->iterators, l.second)});
        n->rhs = lower_expr(build, C, n->iterators, e);
        if (C->get_predicate().is_defined()) n->predicate = lower_expr(build, C, n->iterators, C->get_predicate());
        if (C->get_access_relation()) {
            std::vector<expr> self;
            for (auto &nm : names) self.push_back(var(nm));
            // own store relation: an access to oneself at the current instance
            std::map<std::string, expr> it2 = n->iterators;
            for (auto &nm : names) if (!it2.count(nm)) it2[nm] = expr((int32_t)0);
            expr a = lower_access(build, C, it2, C, self);
            n->lhs = find_buffer(a.get_name());
            n->lhs_index = a.get_access();
        } else if (n->lkind == leaf_kind::assign) {
            ERROR("computation " + C->get_name() + " has no buffer to store its result", true);
        } else if (n->lkind == leaf_kind::let && C->get_predicate().is_defined()) {
            ERROR("constant " + C->get_name() + " cannot carry a predicate", true);
        }
        return n;
    }
};

isl_ast_node *at_each_domain(isl_ast_node *nd, isl_ast_build *build, void *user) {
    lowering *lw = (lowering *)user;
    isl_ast_expr *call = isl_ast_node_user_get_expr(nd);
    isl_ast_expr *a0 = isl_ast_expr_get_op_arg(call, 0);
    isl_id *id = isl_ast_expr_get_id(a0);
    std::string nm = isl_id_get_name(id);
    isl_id_free(id);
    isl_ast_expr_free(a0);
    auto v = lw->f->get_computation_by_name(nm);
    if (v.empty()) ERROR("AST names an unknown computation " + nm, true);
    lw->leaves.push_back(lw->make_leaf(build, v[0], call));
    isl_ast_expr_free(call);
    isl_id *ann = isl_id_alloc(lw->f->get_isl_ctx(), "leaf", (void *)(intptr_t)lw->leaves.size());
    return isl_ast_node_set_annotation(nd, ann);
}

node_ptr convert(lowering &lw, isl_ast_node *nd) {
    node_ptr n = std::make_shared<node>();
    switch (isl_ast_node_get_type(nd)) {
    case isl_ast_node_block: {
        n->kind = node_kind::block;
        isl_ast_node_list *l = isl_ast_node_block_get_children(nd);
        int k = isl_ast_node_list_n_ast_node(l);
        for (int i = 0; i < k; i++) {
            isl_ast_node *c = isl_ast_node_list_get_ast_node(l, i);
            n->children.push_back(convert(lw, c));
            isl_ast_node_free(c);
        }
        isl_ast_node_list_free(l);
        break;
    }
    case isl_ast_node_for: {
        n->kind = node_kind::loop;
        isl_ast_expr *it = isl_ast_node_for_get_iterator(nd);
        isl_id *id = isl_ast_expr_get_id(it);
        n->iterator = isl_id_get_name(id);
        isl_id_free(id);
        isl_ast_expr_free(it);
        if (n->iterator.size() > 1 && n->iterator[0] == 'c') n->level = (std::atoi(n->iterator.c_str() + 1) - 1) / 2;
        isl_ast_expr *init = isl_ast_node_for_get_init(nd);
        n->init = lw.from_isl(init, {});
        isl_ast_expr_free(init);
        isl_ast_expr *inc = isl_ast_node_for_get_inc(nd);
        n->increment = lw.from_isl(inc, {});
        isl_ast_expr_free(inc);
        isl_ast_expr *cond = isl_ast_node_for_get_cond(nd);
        isl_ast_op_type ct = isl_ast_expr_get_op_type(cond);
        isl_ast_expr *ub = isl_ast_expr_get_op_arg(cond, 1);
        expr u = lw.from_isl(ub, {});
        isl_ast_expr_free(ub);
        isl_ast_expr_free(cond);
        if (ct == isl_ast_op_lt) u = lir::simplify(u - 1);
        else if (ct != isl_ast_op_le) ERROR("unexpected loop condition in the isl AST", true);
        n->upper = u;
        isl_ast_node *b = isl_ast_node_for_get_body(nd);
        n->body = convert(lw, b);
        isl_ast_node_free(b);
        break;
    }
    case isl_ast_node_if: {
        n->kind = node_kind::cond;
        isl_ast_expr *c = isl_ast_node_if_get_cond(nd);
        n->condition = lw.from_isl(c, {});
        isl_ast_expr_free(c);
        isl_ast_node *t = isl_ast_node_if_get_then(nd);
        n->then_body = convert(lw, t);
        isl_ast_node_free(t);
        if (isl_ast_node_if_has_else(nd) == isl_bool_true) {
            isl_ast_node *e = isl_ast_node_if_get_else(nd);
            n->else_body = convert(lw, e);
            isl_ast_node_free(e);
        }
        break;
    }
    case isl_ast_node_mark: {
        isl_ast_node *c = isl_ast_node_mark_get_node(nd);
        n = convert(lw, c);
        isl_ast_node_free(c);
        break;
    }
    case isl_ast_node_user: {
        isl_id *ann = isl_ast_node_get_annotation(nd);
        if (!ann) ERROR("statement without annotation in the isl AST", true);
        intptr_t idx = (intptr_t)isl_id_get_user(ann);
        isl_id_free(ann);
        n = lw.leaves.at(idx - 1);
        break;
    }
    default: ERROR("unexpected isl AST node", true);
    }
    return n;
}

void collect_leaves(const node_ptr &n, std::vector<node *> &out) {
    lir::walk(n, [&](const node_ptr &x) { if (x->kind == node_kind::leaf) out.push_back(x.get()); });
}

// A loop carries a tag when any statement below it was tagged at that loop level.
void apply_tags(function *f, const node_ptr &root) {
    lir::walk(root, [&](const node_ptr &n) {
        if (n->kind != node_kind::loop || n->level < 0) return;
        std::vector<node *> leaves;
        collect_leaves(n->body, leaves);
        for (auto l : leaves) {
            const std::string &cn = l->comp->get_name();
            if (f->should_parallelize(cn, n->level)) n->parallel = true;
            if (int v = f->vector_length(cn, n->level)) n->vector_length = v;
            if (f->should_unroll(cn, n->level)) n->unrolled = true;
            int b = f->gpu_block_position(cn, n->level);
            if (b >= 0) n->gpu_block = b;
            int t = f->gpu_thread_position(cn, n->level);
            if (t >= 0) n->gpu_thread = t;
        }
    });
}

// isl leaves no loop node where a loop level has a single iteration, so a statement all of whose tagged levels are of
// that kind (a domain of one point; in general one that fits in a single tile of extent one per tagged dimension)
// would stay on the host with its GPU buffers -- the reference has the same gap ("TODO check if degenerate",
// tiramisu_codegen_cuda.cpp:252).  The largest subtrees that consist of such statements alone become the body of a
// block loop of one iteration, placed inside the loops that lie outside the statements' first tagged level: a kernel
// of one workgroup.
// first loop level at which the statement is tagged for the GPU, -1 when it has no such tag
int first_gpu_level(function *f, const node *leaf) {
    if (!leaf->comp) return -1;
    const std::string &cn = leaf->comp->get_name();
    for (int level = 0; level < 32; level++)
        if (f->gpu_block_position(cn, level) >= 0 || f->gpu_thread_position(cn, level) >= 0) return level;
    return -1;
}

void keep_on_gpu(function *f, node_ptr &n) {
    if (!n) return;
    if (n->kind == node_kind::loop && (n->gpu_block >= 0 || n->gpu_thread >= 0)) return;
    std::vector<node *> leaves;
    collect_leaves(n, leaves);
    bool alone = !leaves.empty();
    int outermost = 32;
    for (auto l : leaves) {
        const int first = first_gpu_level(f, l);
        if (first < 0) alone = false;
        else outermost = std::min(outermost, first);
    }
    // loops outside the statements' first tagged level stay around the kernel (host loops, one launch per iteration)
    lir::walk(n, [&](const node_ptr &x) {
        if (x->kind != node_kind::loop) return;
        if (x->gpu_block >= 0 || x->gpu_thread >= 0 || (x->level >= 0 && x->level < outermost)) alone = false;
    });
    if (alone) {
        node_ptr once = std::make_shared<node>();
        once->kind = node_kind::loop;
        once->iterator = "_single_iteration";
        once->init = expr((int32_t)0);
        once->upper = expr((int32_t)0);
        once->increment = expr((int32_t)1);
        once->gpu_block = 0;
        once->body = n;
        n = once;
        return;
    }
    for (auto &c : n->children) keep_on_gpu(f, c);
    keep_on_gpu(f, n->body);
    keep_on_gpu(f, n->then_body);
    keep_on_gpu(f, n->else_body);
}

}  // namespace

namespace {

// The schedule as a tree (option ast_from_schedule_tree).  The reference hands isl one flat map from statement
// instances to time vectors (tiramisu_function.cpp: gen_isl_ast, isl_ast_build_node_from_schedule_map), and isl then
// finds out, level by level, which statements' domains follow which -- pairwise, an emptiness test each: with the
// hundreds of statements of a tensor-contraction program three quarters of the generation time.  But the time vectors
// say it outright: positions 0, 2, 4, ... hold the statement's place among its siblings (constants), positions 1, 3, ...
// the loops.  So: a sequence node over the groups of equal constant for an even position (none when all agree), a band
// of one member for an odd position, and so on down.  The AST is the same; isl is told the order instead of deriving it.
struct scheduled_statement { isl_map *schedule; isl_pw_multi_aff *time; };

isl_schedule_node *place(isl_ctx *ctx, isl_schedule_node *node, const std::vector<scheduled_statement *> &group, int p, int dims) {
    if (p >= dims) return node;
    if (p % 2 == 0) {
        std::map<long, std::vector<scheduled_statement *>> by_place;
        for (auto s : group) {
            isl_val *v = isl_map_plain_get_val_if_fixed(s->schedule, isl_dim_out, p);
            if (!v || isl_val_is_int(v) != isl_bool_true) { isl_val_free(v); return nullptr; }
            by_place[isl_val_get_num_si(v)].push_back(s);
            isl_val_free(v);
        }
        if (by_place.size() == 1) return place(ctx, node, group, p + 1, dims);
        isl_union_set_list *filters = isl_union_set_list_alloc(ctx, (int)by_place.size());
        for (auto &g : by_place) {
            isl_union_set *members = nullptr;
            for (auto s : g.second) {
                isl_union_set *d = isl_union_set_from_set(isl_map_domain(isl_map_copy(s->schedule)));
                members = members ? isl_union_set_union(members, d) : d;
            }
            filters = isl_union_set_list_add(filters, members);
        }
        node = isl_schedule_node_insert_sequence(node, filters);
        int child = 0;
        for (auto &g : by_place) {
            node = isl_schedule_node_child(isl_schedule_node_child(node, child++), 0);
            node = place(ctx, node, g.second, p + 1, dims);
            if (!node) return nullptr;
            node = isl_schedule_node_parent(isl_schedule_node_parent(node));
        }
        return node;
    }
    // A statement whose coordinate here is a constant while its siblings' are loops (a copy left unordered against
    // a loop nest: same place, no loop of its own) would be scanned inside those loops under a guard; the flat form
    // separates it out, which is what the emitters need (no copy inside a kernel).  Such schedules are left to it.
    int constant = 0;
    for (auto s : group) {
        isl_val *v = isl_map_plain_get_val_if_fixed(s->schedule, isl_dim_out, p);
        if (v && isl_val_is_int(v) == isl_bool_true) constant++;
        isl_val_free(v);
    }
    if (constant != 0 && constant != (int)group.size()) return nullptr;
    isl_union_pw_aff *when = nullptr;
    for (auto s : group) {
        isl_union_pw_aff *u = isl_union_pw_aff_from_pw_aff(isl_pw_multi_aff_get_pw_aff(s->time, p));
        when = when ? isl_union_pw_aff_union_add(when, u) : u;
    }
    node = isl_schedule_node_insert_partial_schedule(node, isl_multi_union_pw_aff_from_union_pw_aff(when));
    node = place(ctx, isl_schedule_node_child(node, 0), group, p + 1, dims);
    return node ? isl_schedule_node_parent(node) : nullptr;
}

}  // namespace

void function::gen_isl_ast() {
    for (auto c : body)
        if (!c->get_time_space_domain()) { gen_time_space_domain(); break; }
    isl_options_set_on_error(ctx, ISL_ON_ERROR_WARN);
    isl_options_set_ast_build_atomic_upper_bound(ctx, 1);
    isl_options_set_ast_build_group_coscheduled(ctx, 1);

    isl_union_map *umap = nullptr;
    for (auto c : body) {
        if (!c->should_schedule_this_computation()) continue;   // function-wide constants, inputs
        isl_map *m = isl_map_copy(c->get_schedule());
        m = isl_map_project_out(m, isl_dim_out, 0, 1);  // the duplicate dimension
        isl_set *d = isl_set_copy(c->get_iteration_domain());
        if (context_set) d = isl_set_intersect_params(d, isl_set_copy(context_set));
        m = isl_map_intersect_domain(m, d);
        isl_union_map *u = isl_union_map_from_map(m);
        umap = umap ? isl_union_map_union(umap, u) : u;
    }
    if (!umap) ERROR("function " + name + " has nothing to schedule", true);

    // "1": build the AST from the schedule as a tree where the schedule has that layout; "check": build it both ways,
    // keep the flat form's and report whether the two programs read the same
    const char *tree_option = backend_option("TIRAMISU_AST_FROM_SCHEDULE_TREE");
    const std::string tree_mode = tree_option ? tree_option : "0";
    isl_schedule *tree = nullptr;
    if (tree_mode != "0") {
        std::vector<scheduled_statement> statements;
        int dims = -1;
        bool uniform = true;
        isl_map_list *maps = isl_union_map_get_map_list(umap);
        for (int i = 0; i < isl_map_list_n_map(maps); i++) {
            isl_map *m = isl_map_list_get_map(maps, i);
            const int nd = isl_map_dim(m, isl_dim_out);
            if (dims >= 0 && nd != dims) uniform = false;
            dims = nd;
            statements.push_back({m, isl_pw_multi_aff_from_map(isl_map_copy(m))});
        }
        isl_map_list_free(maps);
        if (uniform && !statements.empty()) {
            std::vector<scheduled_statement *> all;
            for (auto &s : statements) all.push_back(&s);
            isl_schedule *start = isl_schedule_from_domain(isl_union_map_domain(isl_union_map_copy(umap)));
            isl_schedule_node *root = isl_schedule_get_root(start);
            isl_schedule_free(start);
            isl_schedule_node *done = place(ctx, isl_schedule_node_child(root, 0), all, 0, dims);
            if (done) {
                tree = isl_schedule_node_get_schedule(done);
                isl_schedule_node_free(done);
            }
        }
        for (auto &s : statements) { isl_map_free(s.schedule); isl_pw_multi_aff_free(s.time); }
        if (!tree && debug_level() >= 1) std::cout << "schedule of " << name << " is left to the flat form" << std::endl;
    }
    auto build_ast = [&](lowering &lw, bool from_tree) -> isl_ast_node * {
        isl_ast_build *build = context_set ? isl_ast_build_from_context(isl_set_copy(context_set)) : isl_ast_build_alloc(ctx);
        build = isl_ast_build_set_at_each_domain(build, &at_each_domain, &lw);
        isl_ast_node *result;
        if (from_tree) {
            // loops take the names they have in the flat form, where every position of the time vector has a name
            // and the loops sit at the odd ones: c1, c3, ...
            int dims = 0;
            isl_map_list *maps = isl_union_map_get_map_list(umap);
            if (isl_map_list_n_map(maps) > 0) { isl_map *m = isl_map_list_get_map(maps, 0); dims = isl_map_dim(m, isl_dim_out); isl_map_free(m); }
            isl_map_list_free(maps);
            isl_id_list *names = isl_id_list_alloc(ctx, dims / 2 + 1);
            for (int p = 1; p < dims; p += 2) names = isl_id_list_add(names, isl_id_alloc(ctx, ("c" + std::to_string(p)).c_str(), nullptr));
            build = isl_ast_build_set_iterators(build, names);
            result = isl_ast_build_node_from_schedule(build, isl_schedule_copy(tree));
        } else {
            result = isl_ast_build_node_from_schedule_map(build, isl_union_map_copy(umap));
        }
        isl_ast_build_free(build);
        return result;
    };

    lowering lw;
    lw.f = this;
    const bool use_tree = tree && tree_mode == "1";
    ast = build_ast(lw, use_tree);
    if (!ast) ERROR("isl failed to generate an AST for " + name, true);

    lowered.reset(new lir::program());
    lowered->fct = this;
    lowered->root = convert(lw, ast);
    apply_tags(this, lowered->root);
    keep_on_gpu(this, lowered->root);
    if (tree && tree_mode == "check") {
        lowering other;
        other.f = this;
        isl_ast_node *second = build_ast(other, true);
        if (!second) ERROR("isl failed to generate an AST for " + name + " from the schedule tree", true);
        node_ptr root2 = convert(other, second);
        apply_tags(this, root2);
        keep_on_gpu(this, root2);
        isl_ast_node_free(second);
        const std::string a = lir::dump(lowered->root), b = lir::dump(root2);
        if (a != b) std::cerr << "---- from the schedule map\n" << a << "---- from the schedule tree\n" << b
                              << "schedule tree check: " << name << " gives another program text than its schedule map" << std::endl;
        else std::cerr << "schedule tree check: " << name << " gives the same program both ways" << std::endl;
    } else if (tree_mode == "check") {
        std::cerr << "schedule tree check: " << name << " is left to the flat form" << std::endl;
    }
    if (tree) isl_schedule_free(tree);
    isl_union_map_free(umap);

    // Function-wide constants: literal-indexed reads of argument buffers, or plain expressions.
    for (auto c : invariants) {
        lir::invariant inv;
        inv.name = c->get_name();
        inv.type = c->get_data_type();
        inv.value = c->get_expr().transform([&](const expr &e) -> expr {
            if (e.get_expr_type() != e_op || e.get_op_type() != o_access) return e;
            computation *X = lw.find_computation(e.get_name());
            if (!X) ERROR("constant " + c->get_name() + " reads unknown computation " + e.get_name(), true);
            if (X->is_let_stmt()) return var(X->get_data_type(), X->get_name());
            isl_map *m = isl_map_copy(X->get_access_relation());
            for (size_t i = 0; i < e.get_access().size(); i++) {
                expr a = lir::simplify(e.get_access()[i]);
                if (!a.is_integer_literal())
                    ERROR("constant " + c->get_name() + ": only literal indices are supported in its definition", true);
                m = isl_map_fix_si(m, isl_dim_in, i, (int)a.get_int_val());
            }
            std::vector<expr> idx;
            int nd = isl_map_dim(m, isl_dim_out);
            for (int d = 0; d < nd; d++) {
                isl_val *v = isl_map_plain_get_val_if_fixed(m, isl_dim_out, d);
                if (!v || isl_val_is_int(v) != isl_bool_true)
                    ERROR("constant " + c->get_name() + ": cannot resolve the buffer element it reads", true);
                idx.push_back(expr((int32_t)isl_val_get_num_si(v)));
                isl_val_free(v);
            }
            std::string bn = isl_map_get_tuple_name(m, isl_dim_out);
            isl_map_free(m);
            return expr(o_access, bn, idx, X->get_data_type());
        });
        lowered->invariants.push_back(inv);
    }
    if (debug_level() >= 1) std::cout << lir::dump(lowered->root) << std::endl;
}

namespace lir {

expr extent_of_dimension(function *f, isl_set *domain, int d) {
    isl_pw_aff *largest = isl_set_dim_max(isl_set_copy(domain), d);
    isl_ast_build *build = isl_ast_build_from_context(isl_set_params(isl_set_copy(domain)));
    isl_ast_expr *e = isl_ast_build_expr_from_pw_aff(build, largest);
    lowering L;
    L.f = f;
    expr r = simplify(L.from_isl(e, {}) + value_cast(global::get_loop_iterator_data_type(), 1));
    isl_ast_expr_free(e);
    isl_ast_build_free(build);
    return r;
}

node_ptr canonical_nest(function &f, computation &c, bool as_written) {
    isl_ctx *ctx = f.get_isl_ctx();
    int n = isl_set_dim(c.get_iteration_domain(), isl_dim_set);
    std::vector<std::string> in;
    for (int i = 0; i < n; i++) in.push_back("t" + std::to_string(i));
    std::string ms = "{ " + c.get_name() + "[" + join(in, ",") + "] -> [" + join(in, ",") + "] }";
    isl_map *m = isl_map_read_from_str(ctx, ms.c_str());
    isl_set *d = isl_set_copy(c.get_iteration_domain());
    if (f.get_program_context()) d = isl_set_intersect_params(d, isl_set_copy(f.get_program_context()));
    m = isl_map_intersect_domain(m, d);
    lowering lw;
    lw.f = &f;
    lw.as_written = as_written;
    isl_ast_build *build = f.get_program_context() ? isl_ast_build_from_context(isl_set_copy(f.get_program_context()))
                                                   : isl_ast_build_alloc(ctx);
    build = isl_ast_build_set_at_each_domain(build, &at_each_domain, &lw);
    isl_ast_node *ast = isl_ast_build_node_from_schedule_map(build, isl_union_map_from_map(m));
    isl_ast_build_free(build);
    if (!ast) return nullptr;
    node_ptr root = convert(lw, ast);
    isl_ast_node_free(ast);
    return root;
}

bool mentions(const expr &e, const std::string &v) {
    bool m = false;
    e.visit([&](const expr &x) { if (x.get_expr_type() == e_var && x.get_name() == v) m = true; });
    return m;
}

expr coefficient(const expr &e, const std::string &v, bool &ok) {
    primitive_t t = global::get_loop_iterator_data_type();
    const expr zero = value_cast(t, (int64_t)0), one = value_cast(t, (int64_t)1);
    if (!mentions(e, v)) return zero;
    switch (e.get_expr_type()) {
    case e_var: return one;
    case e_op:
        switch (e.get_op_type()) {
        case o_add: return simplify(coefficient(e.get_operand(0), v, ok) + coefficient(e.get_operand(1), v, ok));
        case o_sub: return simplify(coefficient(e.get_operand(0), v, ok) - coefficient(e.get_operand(1), v, ok));
        case o_minus: return simplify(zero - coefficient(e.get_operand(0), v, ok));
        case o_cast: return is_int_type(e.get_data_type()) ? coefficient(e.get_operand(0), v, ok) : (ok = false, zero);
        case o_mul: {
            const expr &a = e.get_operand(0), &b = e.get_operand(1);
            if (!mentions(a, v)) return simplify(cast(t, a) * coefficient(b, v, ok));
            if (!mentions(b, v)) return simplify(coefficient(a, v, ok) * cast(t, b));
            ok = false;
            return zero;
        }
        default: ok = false; return zero;
        }
    default: ok = false; return zero;
    }
}

}  // namespace lir

void function::gen_c_code() const {
    char *s = isl_ast_node_to_C_str(ast);
    std::cout << s << std::endl;
    free(s);
}

// ------------------------------------------------------------------ lir helpers

namespace lir {

expr simplify(const expr &e) {
    if (!e.is_defined() || e.get_expr_type() != e_op) return e;
    op_t o = e.get_op_type();
    if (e.get_n_arg() == 2 && (o == o_add || o == o_sub || o == o_mul || o == o_div || o == o_mod)) {
        expr a = simplify(e.get_operand(0)), b = simplify(e.get_operand(1));
        primitive_t t = e.get_data_type();
        if (is_int_type(t) && a.is_integer_literal() && b.is_integer_literal()) {
            int64_t x = a.get_int_val(), y = b.get_int_val();
            switch (o) {
            case o_add: return value_cast(t, x + y);
            case o_sub: return value_cast(t, x - y);
            case o_mul: return value_cast(t, x * y);
            case o_div: if (y != 0 && x >= 0 && y > 0) return value_cast(t, x / y); break;
            case o_mod: if (y != 0 && x >= 0 && y > 0) return value_cast(t, x % y); break;
            default: break;
            }
        }
        if (is_int_type(t)) {
            auto lit = [](const expr &x, int64_t v) { return x.is_integer_literal() && x.get_int_val() == v; };
            if (o == o_add && lit(a, 0)) return b;
            if ((o == o_add || o == o_sub) && lit(b, 0)) return a;
            if (o == o_mul && (lit(a, 0) || lit(b, 0))) return value_cast(t, (int64_t)0);
            if (o == o_mul && lit(a, 1)) return b;
            if ((o == o_mul || o == o_div) && lit(b, 1)) return a;
        }
        return expr(o, a, b).copy_with_type(t);
    }
    return e;
}

expr linearize(const buffer *b, const std::vector<expr> &index) {
    const auto &sizes = b->get_dim_sizes();
    if (index.size() != sizes.size())
        ERROR("access to buffer " + b->get_name() + " with " + std::to_string(index.size()) + " indices, it has " +
              std::to_string(sizes.size()) + " dimensions", true);
    primitive_t it = global::get_loop_iterator_data_type();
    expr lin;
    for (size_t d = 0; d < index.size(); d++) {
        expr term = cast(it, index[d]);
        for (size_t k = d + 1; k < sizes.size(); k++) term = simplify(term * cast(it, sizes[k]));
        lin = lin.is_defined() ? simplify(lin + term) : term;
    }
    return lin.is_defined() ? lin : expr((int32_t)0);
}

std::string dump(const node_ptr &n, int indent) {
    if (!n) return "";
    std::ostringstream os;
    std::string pad(indent * 2, ' ');
    switch (n->kind) {
    case node_kind::block:
        for (auto &c : n->children) os << dump(c, indent);
        break;
    case node_kind::loop:
        os << pad << "for " << n->iterator << " = " << n->init.to_str() << " .. " << n->upper.to_str();
        if (n->parallel) os << " [parallel]";
        if (n->vector_length) os << " [vector " << n->vector_length << "]";
        if (n->unrolled) os << " [unroll]";
        if (n->gpu_block >= 0) os << " [block." << "xyz"[n->gpu_block] << "]";
        if (n->gpu_thread >= 0) os << " [thread." << "xyz"[n->gpu_thread] << "]";
        os << "\n" << dump(n->body, indent + 1);
        break;
    case node_kind::cond:
        os << pad << "if " << n->condition.to_str() << "\n" << dump(n->then_body, indent + 1);
        if (n->else_body) os << pad << "else\n" << dump(n->else_body, indent + 1);
        break;
    case node_kind::leaf:
        os << pad;
        switch (n->lkind) {
        case leaf_kind::sync: os << "sync"; break;
        case leaf_kind::copy: os << "copy " << n->copy_from->get_name() << " -> " << n->copy_to->get_name(); break;
        case leaf_kind::allocate: os << "allocate " << n->target->get_name(); break;
        case leaf_kind::release: os << "free " << n->target->get_name(); break;
        case leaf_kind::let: os << "let " << n->comp->get_name(); break;
        default:
            if (n->predicate.is_defined()) os << "if " << n->predicate.to_str() << ": ";
            if (n->lhs) os << expr(o_access, n->lhs->get_name(), n->lhs_index, p_none).to_str() << " = ";
            os << n->rhs.to_str();
        }
        os << "   // " << n->comp->get_name() << "\n";
        break;
    }
    return os.str();
}

}  // namespace lir
}  // namespace tiramisu
