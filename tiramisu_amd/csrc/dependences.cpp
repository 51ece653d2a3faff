// Dependence analysis over buffers and the legality checks built on it (the calls of the reference's
// core.h:139-181, :1236-1330, :4466-4483; its implementation is tiramisu_function.cpp:165-357, :2618-3660 and
// tiramisu_core.cpp:4695-5011).
//
// A dependence is kept as isl's dataflow analysis gives it, { source -> [sink -> cell] } over iteration domains,
// which no later schedule command changes.  A schedule is legal when it maps every source strictly before its
// sink in the time-space order, so every check here is one emptiness test on
//     dependences, mapped through the schedules on both sides, intersected with { a -> b : a >=lex b }.
#include <tiramisu/core.h>

#include <algorithm>
#include <cstdlib>
#include <map>

#include <tiramisu/isl_api.h>
#include "util.h"

namespace tiramisu {

namespace {

isl_union_map *empty_union_map(isl_ctx *ctx) { return isl_union_map_read_from_str(ctx, "{}"); }

void unite(isl_union_map *&into, isl_map *m) {
    if (m) into = isl_union_map_union(into, isl_union_map_from_map(m));
}

// { instance -> time } of the computations given, over their iteration domains
isl_union_map *schedules_of(isl_ctx *ctx, const std::vector<computation *> &comps) {
    isl_union_map *all = empty_union_map(ctx);
    for (auto c : comps)
        if (c->get_schedule()) unite(all, isl_map_intersect_domain(isl_map_copy(c->get_schedule()), isl_set_copy(c->get_iteration_domain())));
    return all;
}

// { time of the source -> time of the sink } for the dependences whose source is scheduled by `from` and whose sink by `to`;
// null when there is none
isl_map *in_time(isl_union_map *deps, isl_union_map *from, isl_union_map *to) {
    isl_union_map *t = isl_union_map_apply_range(isl_union_map_apply_domain(deps, from), to);
    if (isl_union_map_is_empty(t) == isl_bool_true) {
        isl_union_map_free(t);
        return nullptr;
    }
    return isl_map_from_union_map(t);           // one space: the schedules are aligned
}

// the pairs of `t` whose source does not come strictly first
isl_map *out_of_order(isl_map *t) {
    isl_map *ge = isl_map_lex_ge(isl_space_range(isl_map_get_space(t)));
    return isl_map_intersect(t, ge);
}

bool none_out_of_order(isl_map *t) {
    if (!t) return true;
    isl_map *bad = out_of_order(t);
    const bool ok = isl_map_is_empty(bad) == isl_bool_true;
    isl_map_free(bad);
    return ok;
}

// whether a dependence (in time, may be null) links two iterations of the loop at time dimension `at` inside one
// iteration of the loops around it
bool carried_by(isl_map *t, int at) {
    if (!t) return false;
    for (int d = 0; d < at; d++) t = isl_map_equate(t, isl_dim_in, d, isl_dim_out, d);
    isl_map *within = isl_map_equate(isl_map_copy(t), isl_dim_in, at, isl_dim_out, at);
    isl_map *carried = isl_map_subtract(t, within);
    const bool yes = isl_map_is_empty(carried) != isl_bool_true;
    isl_map_free(carried);
    return yes;
}

void need_analysis(const function *f) {
    if (!f->dep_read_after_write || !f->dep_write_after_read || !f->dep_write_after_write)
        ERROR("legality checks need perform_full_dependency_analysis() first", true);
}

}  // namespace

// ------------------------------------------------------------------ the analysis

void function::calculate_dep_flow(bool global_memory_only) {
    for (isl_union_map **m : {&dep_read_after_write, &dep_write_after_read, &dep_write_after_write, &live_in_access, &live_out_access}) {
        if (*m) isl_union_map_free(*m);
        *m = nullptr;
    }
    std::vector<computation *> scheduled;
    for (auto c : body)
        if (c->should_schedule_this_computation() && c->get_schedule() && !c->is_inline_computation()) scheduled.push_back(c);
    isl_union_map *schedule = schedules_of(ctx, scheduled);
    isl_union_map *writes = empty_union_map(ctx), *reads = empty_union_map(ctx);
    // with global_memory_only, accesses to LDS, registers and constant memory stay out: what goes through them is
    // ordered by barriers (or private to a thread), not by the loops
    auto counted = [&](computation *c) {
        if (!c->get_access_relation()) return false;
        if (!global_memory_only) return true;
        const char *b = isl_map_get_tuple_name(c->get_access_relation(), isl_dim_out);
        auto it = b ? buffers_list.find(b) : buffers_list.end();
        return it == buffers_list.end() || it->second->location == memory_location::host || it->second->location == memory_location::global;
    };
    for (auto c : scheduled) {
        if (counted(c))
            unite(writes, isl_map_intersect_domain(isl_map_copy(c->get_access_relation()), isl_set_copy(c->get_iteration_domain())));
        // what c reads of p, carried on to the cells p is stored in (an input writes nothing here but is read from its buffer)
        for (auto p : body) {
            if (!counted(p)) continue;
            isl_map *r = reads_of(*c, *p, false, true);
            if (r) unite(reads, isl_map_apply_range(r, isl_map_copy(p->get_access_relation())));
        }
    }
    // (not coalesced: two reads at constant distances must not merge into one relation with a range of distances)

    auto flow_of = [&](isl_union_map *sink, isl_union_map *must, isl_union_map *may, isl_union_map *kill) {
        isl_union_access_info *info = isl_union_access_info_from_sink(sink);
        info = isl_union_access_info_set_schedule_map(info, isl_union_map_copy(schedule));
        if (must) info = isl_union_access_info_set_must_source(info, must);
        if (may) info = isl_union_access_info_set_may_source(info, may);
        if (kill) info = isl_union_access_info_set_kill(info, kill);
        isl_union_flow *flow = isl_union_access_info_compute_flow(info);
        if (!flow) ERROR("dependence analysis failed", true);
        return flow;
    };
    // the last write before every read; reads that see no write are live-in
    isl_union_flow *flow = flow_of(isl_union_map_copy(reads), isl_union_map_copy(writes), nullptr, nullptr);
    dep_read_after_write = isl_union_flow_get_full_must_dependence(flow);
    live_in_access = isl_union_flow_get_must_no_source(flow);
    isl_union_flow_free(flow);
    // the last write before every write; a write that is the source of none is live-out
    flow = flow_of(isl_union_map_copy(writes), isl_union_map_copy(writes), nullptr, nullptr);
    dep_write_after_write = isl_union_flow_get_full_must_dependence(flow);
    isl_union_flow_free(flow);
    live_out_access = isl_union_map_subtract(isl_union_map_copy(writes), isl_union_map_range_factor_range(isl_union_map_copy(dep_write_after_write)));
    // every read before a write of the same cell, unless another write lies between them; an instance that
    // reads the cell it writes does not depend on itself
    isl_union_map *reads_elsewhere = isl_union_map_subtract(isl_union_map_copy(reads), isl_union_map_copy(writes));
    flow = flow_of(isl_union_map_copy(writes), nullptr, reads_elsewhere, isl_union_map_copy(writes));
    dep_write_after_read = isl_union_flow_get_full_may_dependence(flow);
    isl_union_flow_free(flow);
    isl_union_map_free(schedule);
    isl_union_map_free(writes);
    isl_union_map_free(reads);
}

void function::perform_full_dependency_analysis() {
    align_schedules();
    gen_ordering_schedules();
    calculate_dep_flow();
}

isl_union_map *function::get_statement_dependences() const {
    need_analysis(this);
    isl_union_map *all = isl_union_map_range_factor_domain(isl_union_map_copy(dep_read_after_write));
    all = isl_union_map_union(all, isl_union_map_range_factor_domain(isl_union_map_copy(dep_write_after_read)));
    return isl_union_map_union(all, isl_union_map_range_factor_domain(isl_union_map_copy(dep_write_after_write)));
}

std::string function::dependences_as_text() const {
    need_analysis(this);
    std::string text;
    const std::pair<const char *, isl_union_map *> parts[] = {{"read_after_write", dep_read_after_write}, {"write_after_read", dep_write_after_read},
                                                              {"write_after_write", dep_write_after_write}, {"live_in", live_in_access}, {"live_out", live_out_access}};
    for (auto &p : parts) {
        isl_union_map *m = isl_union_map_coalesce(isl_union_map_copy(p.second));
        char *s = isl_union_map_to_str(m);
        text += std::string(p.first) + ": " + (s ? s : "?") + "\n";
        free(s);
        isl_union_map_free(m);
    }
    return text;
}

void function::reset_all_static_dims_to_zero() {
    for (auto c : body) {
        if (!c->get_schedule()) continue;
        const int n = (int)isl_map_dim(c->get_schedule(), isl_dim_out);
        std::vector<std::string> in, out;
        for (int i = 0; i < n; i++) {
            in.push_back("x" + std::to_string(i));
            out.push_back(i == 0 || i % 2 == 1 ? std::string("0") : in.back());     // the duplicate number and the static dimensions
        }
        c->apply_on_range("{ [" + join(in, ",") + "] -> [" + join(out, ",") + "] }");
    }
}

void function::prepare_schedules_for_legality_checks(bool reset_static_dimesion) {
    align_schedules();
    if (reset_static_dimesion) reset_all_static_dims_to_zero();
    gen_ordering_schedules();
}

// ------------------------------------------------------------------ order of sources and sinks

bool function::check_partial_legality_in_function(std::vector<computation *> involved_computations) {
    isl_union_map *deps = get_statement_dependences();
    isl_union_map *s = schedules_of(ctx, involved_computations);
    return none_out_of_order(in_time(deps, isl_union_map_copy(s), s));
}

bool function::check_legality_for_function() {
    std::vector<computation *> all;
    for (auto c : body)
        if (c->should_schedule_this_computation()) all.push_back(c);
    return check_partial_legality_in_function(all);
}

bool computation::involved_subset_of_dependencies_is_legal(computation *second) {
    isl_union_map *deps = fct->get_statement_dependences();
    return none_out_of_order(in_time(deps, schedules_of(ctx, {this}), schedules_of(ctx, {second})));
}

// ------------------------------------------------------------------ one loop

bool function::loop_parallelization_is_legal(int parallel_dim, std::vector<computation *> fused_computations) {
    if (fused_computations.empty()) ERROR("loop_parallelization_is_legal: no computation given", true);
    isl_union_map *s = schedules_of(ctx, fused_computations);
    return !carried_by(in_time(get_statement_dependences(), isl_union_map_copy(s), s), fused_computations[0]->dynamic_pos(parallel_dim));
}

bool function::loop_parallelization_is_legal(var i, std::vector<computation *> fused_computations) {
    if (fused_computations.empty()) ERROR("loop_parallelization_is_legal: no computation given", true);
    return loop_parallelization_is_legal(fused_computations[0]->get_loop_level_number_from_dimension_name(i.get_name()), fused_computations);
}

bool computation::unrolling_is_legal(var l) {
    const int at = dynamic_pos(get_loop_level_number_from_dimension_name(l.get_name()));
    isl_set *time = isl_map_range(isl_map_intersect_domain(isl_map_copy(schedule), isl_set_copy(iteration_domain)));
    const int n = (int)isl_set_dim(time, isl_dim_set);
    if (at >= n) ERROR("unrolling_is_legal: no such loop level in " + name, true);
    time = isl_set_project_out(time, isl_dim_set, at + 1, n - at - 1);
    // one iteration of the loops around, named by parameters
    std::vector<std::string> outer;
    for (int d = 0; d < at; d++) outer.push_back("_o" + std::to_string(d));
    std::vector<std::string> point = outer;
    point.push_back("x");
    isl_set *one = isl_set_read_from_str(ctx, ("[" + join(outer, ",") + "] -> { [" + join(point, ",") + "] }").c_str());
    time = isl_set_intersect(time, one);
    isl_pw_aff *hi = isl_set_dim_max(isl_set_copy(time), at), *lo = isl_set_dim_min(time, at);
    const bool ok = hi && lo && isl_pw_aff_n_piece(hi) == 1 && isl_pw_aff_n_piece(lo) == 1;
    isl_pw_aff_free(hi);
    isl_pw_aff_free(lo);
    return ok;
}

bool function::loop_unrolling_is_legal(var i, std::vector<computation *> fused_computations) {
    if (fused_computations.empty()) ERROR("loop_unrolling_is_legal: no computation given", true);
    need_analysis(this);
    for (auto c : fused_computations)
        if (!c->unrolling_is_legal(i)) return false;
    return true;
}

bool function::loop_vectorization_is_legal(var i, std::vector<computation *> fused_computations) {
    return loop_unrolling_is_legal(i, fused_computations) && loop_parallelization_is_legal(i, fused_computations);
}

// ------------------------------------------------------------------ loops mapped to the GPU

std::vector<std::string> function::gpu_mapped_loops_that_carry_dependences() {
    // the analysis of the program as it is scheduled now, kept apart from the one the program may have asked for
    isl_union_map *kept[5] = {dep_read_after_write, dep_write_after_read, dep_write_after_write, live_in_access, live_out_access};
    dep_read_after_write = dep_write_after_read = dep_write_after_write = live_in_access = live_out_access = nullptr;
    align_schedules();
    calculate_dep_flow(true);
    std::vector<computation *> all;
    for (auto c : body)
        if (c->should_schedule_this_computation() && c->get_schedule() && !c->is_inline_computation()) all.push_back(c);
    // the computations inside the same loop as c at a level: the ordering dimensions before it agree
    auto static_value = [](computation *q, int pos) {
        isl_val *v = isl_map_plain_get_val_if_fixed(q->get_schedule(), isl_dim_out, pos);
        const long value = (v && isl_val_is_int(v) == isl_bool_true) ? isl_val_get_num_si(v) : -1;
        isl_val_free(v);
        return value;
    };
    // a computation that only ever reads, of itself, the cell it is writing: an accumulation.  Its dependences
    // on itself are those of a reduction, which the back-end lowers as one where the loop is mapped
    auto accumulates = [&](computation *c) {
        isl_map *self = c->get_access_relation() ? reads_of(*c, *c, false) : nullptr;
        if (!self) return false;
        isl_map *cells = isl_map_apply_range(self, isl_map_copy(c->get_access_relation()));
        isl_map *own = isl_map_intersect_domain(isl_map_copy(c->get_access_relation()), isl_set_copy(c->get_iteration_domain()));
        const bool yes = isl_map_is_subset(cells, own) == isl_bool_true;
        isl_map_free(cells);
        isl_map_free(own);
        return yes;
    };
    std::vector<std::string> found;
    for (auto c : all) {
        const int levels = (int)c->get_loop_level_names().size();
        for (int l = 0; l < levels; l++) {
            const bool block = gpu_block_position(c->get_name(), l) >= 0, thread = gpu_thread_position(c->get_name(), l) >= 0;
            if (!block && !thread) continue;
            std::vector<computation *> fused;
            for (auto q : all) {
                bool same = true;
                for (int pos = 1; pos < c->dynamic_pos(l) && same; pos += 2) same = static_value(q, pos) == static_value(c, pos);
                if (same) fused.push_back(q);
            }
            if (loop_parallelization_is_legal(l, fused)) continue;
            // a second look without the reductions
            isl_union_map *everything = get_statement_dependences(), *reductions = empty_union_map(ctx);
            for (auto q : fused)
                if (accumulates(q)) {
                    isl_union_set *d = isl_union_set_from_set(isl_set_copy(q->get_iteration_domain()));
                    reductions = isl_union_map_union(reductions, isl_union_map_intersect_range(isl_union_map_intersect_domain(isl_union_map_copy(everything), isl_union_set_copy(d)), d));
                }
            isl_union_map *s = schedules_of(ctx, fused);
            const bool only_reductions = carried_by(in_time(isl_union_map_subtract(everything, reductions), isl_union_map_copy(s), s), c->dynamic_pos(l)) == false;
            found.push_back(c->get_name() + ": loop " + c->get_loop_level_names()[l] + " (level " + std::to_string(l) + ", mapped to " +
                            (block ? "blockIdx" : "threadIdx") + ") carries " + (only_reductions ? "a reduction" : "a dependence") + " through global memory");
        }
    }
    isl_union_map **mine[5] = {&dep_read_after_write, &dep_write_after_read, &dep_write_after_write, &live_in_access, &live_out_access};
    for (int i = 0; i < 5; i++) {
        if (*mine[i]) isl_union_map_free(*mine[i]);
        *mine[i] = kept[i];
    }
    return found;
}

// ------------------------------------------------------------------ shifting a fused computation

std::vector<std::tuple<var, int>> function::correcting_loop_fusion_with_shifting(std::vector<computation *> previous_computations,
                                                                                computation &current,
                                                                                std::vector<var> vars_subjected_to_shifting) {
    std::vector<std::tuple<var, int>> none;
    if (previous_computations.empty() || vars_subjected_to_shifting.empty()) return none;
    // the time dimensions of the loops that may be shifted, outer first
    std::vector<std::pair<int, var>> dims;
    for (auto &v : vars_subjected_to_shifting) dims.push_back({current.dynamic_pos(current.get_loop_level_number_from_dimension_name(v.get_name())), v});
    std::sort(dims.begin(), dims.end(), [](const std::pair<int, var> &a, const std::pair<int, var> &b) { return a.first < b.first; });
    const int innermost = dims.back().first, k = (int)dims.size();
    const int m = (int)isl_map_dim(current.get_schedule(), isl_dim_out);

    isl_union_map *deps = get_statement_dependences();
    isl_union_map *before = schedules_of(ctx, previous_computations), *mine = schedules_of(ctx, {&current});
    isl_map *to_me = in_time(isl_union_map_copy(deps), isl_union_map_copy(before), isl_union_map_copy(mine));
    isl_map *from_me = in_time(deps, mine, before);

    // a shift can only repair distances that are constant down to the innermost shifted loop (and the ordering
    // dimension behind it), piece by piece
    bool constant = true;
    auto check_piece = [](isl_basic_map *piece, void *user) -> isl_stat {
        auto *st = static_cast<std::pair<bool *, int> *>(user);
        isl_set *delta = isl_map_deltas(isl_map_from_basic_map(piece));
        const int n = (int)isl_set_dim(delta, isl_dim_set);
        if (st->second < n) delta = isl_set_project_out(delta, isl_dim_set, st->second, n - st->second);
        if (isl_set_is_singleton(delta) != isl_bool_true) *st->first = false;
        isl_set_free(delta);
        return isl_stat_ok;
    };
    std::pair<bool *, int> state{&constant, innermost + 2};
    for (isl_map *t : {to_me, from_me})
        if (t) isl_map_foreach_basic_map(t, check_piece, &state);
    if (!constant) {
        if (to_me) isl_map_free(to_me);
        if (from_me) isl_map_free(from_me);
        return none;
    }

    // { time -> time shifted by the parameters _n0 ... } and the shifts under which a dependence is out of order
    std::vector<std::string> shifts, x, y;
    for (int i = 0; i < k; i++) shifts.push_back("_n" + std::to_string(i));
    for (int d = 0; d < m; d++) {
        x.push_back("x" + std::to_string(d));
        y.push_back(x.back());
    }
    for (int i = 0; i < k; i++) y[dims[i].first] += " + " + shifts[i];
    const std::string shift_text = "[" + join(shifts, ",") + "] -> { [" + join(x, ",") + "] -> [" + join(y, ",") + "] }";
    std::vector<std::string> bind;
    for (int i = 0; i < k; i++) bind.push_back("a" + std::to_string(i) + " = " + shifts[i]);
    std::vector<std::string> a;
    for (int i = 0; i < k; i++) a.push_back("a" + std::to_string(i));
    isl_set *refused = nullptr;
    auto refuse = [&](isl_map *shifted) {
        isl_set *at = isl_map_params(out_of_order(shifted));
        // as a set over the shifts, for any value of the program's own parameters
        isl_set *s = isl_set_read_from_str(ctx, ("[" + join(shifts, ",") + "] -> { [" + join(a, ",") + "] : " + join(bind, " and ") + " }").c_str());
        s = isl_set_intersect_params(s, at);
        s = isl_set_project_out(s, isl_dim_param, 0, isl_set_dim(s, isl_dim_param));
        refused = refused ? isl_set_union(refused, s) : s;
    };
    if (to_me) refuse(isl_map_apply_range(to_me, isl_map_read_from_str(ctx, shift_text.c_str())));
    if (from_me) refuse(isl_map_apply_domain(from_me, isl_map_read_from_str(ctx, shift_text.c_str())));
    std::vector<std::string> positive;
    for (auto &ai : a) positive.push_back(ai + " >= 0");
    isl_set *allowed = isl_set_read_from_str(ctx, ("{ [" + join(a, ",") + "] : " + join(positive, " and ") + " }").c_str());
    if (refused) allowed = isl_set_subtract(allowed, refused);
    allowed = isl_set_lexmin(allowed);
    std::vector<std::tuple<var, int>> result;
    if (isl_set_is_empty(allowed) != isl_bool_true) {
        for (int i = 0; i < k; i++) {
            isl_val *v = isl_set_dim_min_val(isl_set_copy(allowed), i);
            if (!v || isl_val_is_int(v) != isl_bool_true) {
                isl_val_free(v);
                result.clear();
                break;
            }
            result.push_back(std::make_tuple(dims[i].second, (int)isl_val_get_num_si(v)));
            isl_val_free(v);
        }
    }
    isl_set_free(allowed);
    return result;
}

// ------------------------------------------------------------------ skewing two loops

namespace {

// the distances { [di, dj] } of the dependences at two loop levels, between instances inside one iteration of the
// loops around them, without (0, 0); null when there is none
isl_set *distances_at(function *f, const std::vector<computation *> &fused, int outer, int inner) {
    isl_union_map *s = schedules_of(f->get_isl_ctx(), fused);
    isl_map *t = in_time(f->get_statement_dependences(), isl_union_map_copy(s), s);
    if (!t) return nullptr;
    for (int d = 0; d < outer; d++) t = isl_map_equate(t, isl_dim_in, d, isl_dim_out, d);
    isl_set *delta = isl_map_deltas(t);
    const int n = (int)isl_set_dim(delta, isl_dim_set);
    delta = isl_set_project_out(delta, isl_dim_set, inner + 1, n - inner - 1);
    delta = isl_set_project_out(delta, isl_dim_set, outer + 1, inner - outer - 1);
    delta = isl_set_project_out(delta, isl_dim_set, 0, outer);
    delta = isl_set_project_out(delta, isl_dim_param, 0, isl_set_dim(delta, isl_dim_param));
    delta = isl_set_subtract(delta, isl_set_read_from_str(f->get_isl_ctx(), "{ [0, 0] }"));
    if (isl_set_is_empty(delta) == isl_bool_true) {
        isl_set_free(delta);
        return nullptr;
    }
    return delta;
}

// no distance satisfies the condition (text over di, dj)
bool none(isl_set *delta, const std::string &condition) {
    isl_set *c = isl_set_read_from_str(isl_set_get_ctx(delta), ("{ [di, dj] : " + condition + " }").c_str());
    c = isl_set_intersect(c, isl_set_copy(delta));
    const bool yes = isl_set_is_empty(c) == isl_bool_true;
    isl_set_free(c);
    return yes;
}

std::string row(int a, int b) { return std::to_string(a) + "*di " + (b < 0 ? "- " : "+ ") + std::to_string(std::abs(b)) + "*dj"; }

int common_divisor(int a, int b) {
    a = std::abs(a);
    b = std::abs(b);
    while (b) { const int r = a % b; a = b; b = r; }
    return a;
}

const int LARGEST_COEFFICIENT = 8;

// (a, b), a >= 1, b of the sign given, smallest first
std::vector<std::pair<int, int>> candidates(int sign) {
    std::vector<std::pair<int, int>> v;
    for (int a = 1; a <= LARGEST_COEFFICIENT; a++)
        for (int b = 1; b <= LARGEST_COEFFICIENT; b++)
            if (common_divisor(a, b) == 1) v.push_back({a, sign * b});
    return v;
}

}  // namespace

std::tuple<std::vector<std::pair<int, int>>, std::vector<std::pair<int, int>>, std::vector<std::pair<int, int>>>
function::skewing_local_solver(std::vector<computation *> fused_computations, var outer_variable, var inner_variable, int nb_parallel) {
    std::vector<std::pair<int, int>> outermost, innermost, locality;
    if (fused_computations.empty()) ERROR("skewing_local_solver: no computation given", true);
    computation *c = fused_computations[0];
    const int outer = c->dynamic_pos(c->get_loop_level_number_from_dimension_name(outer_variable.get_name()));
    const int inner = c->dynamic_pos(c->get_loop_level_number_from_dimension_name(inner_variable.get_name()));
    align_schedules();
    isl_set *delta = distances_at(this, fused_computations, outer, inner);
    if (!delta) return std::make_tuple(outermost, innermost, locality);
    for (int sign : {1, -1}) {
        int found = 0;
        bool local = false;
        for (auto &ab : candidates(sign)) {
            const std::string across = row(ab.first, ab.second);
            if (!none(delta, across + " < 0")) continue;                 // some dependence would run backwards in the outer loop
            const bool strongly = none(delta, across + " = 0"), all_inside = none(delta, across + " > 0");
            if (strongly && found < nb_parallel) {                       // the outer loop carries everything: the inner one is free
                innermost.push_back(ab);
                found++;
            }
            int a = ab.first, b = ab.second, gamma, sigma;
            if (all_inside && outermost.empty() && skewing_second_row(a, b, gamma, sigma) && none(delta, row(gamma, sigma) + " <= 0"))
                outermost.push_back(ab);                                  // nothing crosses iterations of the outer loop
            if (!strongly && !all_inside && !local) {
                locality.push_back(ab);
                local = true;
            }
        }
    }
    isl_set_free(delta);
    return std::make_tuple(outermost, innermost, locality);
}

std::tuple<std::vector<std::tuple<int, int, int, int>>, std::vector<std::tuple<int, int, int, int>>, std::vector<std::tuple<int, int, int, int>>>
function::skewing_local_solver_positive(std::vector<computation *> fused_computations, var outer_variable, var inner_variable, int nb_parallel) {
    std::vector<std::tuple<int, int, int, int>> outermost, innermost, identity;
    if (fused_computations.empty()) ERROR("skewing_local_solver_positive: no computation given", true);
    computation *c = fused_computations[0];
    const int outer = c->dynamic_pos(c->get_loop_level_number_from_dimension_name(outer_variable.get_name()));
    const int inner = c->dynamic_pos(c->get_loop_level_number_from_dimension_name(inner_variable.get_name()));
    align_schedules();
    isl_set *delta = distances_at(this, fused_computations, outer, inner);
    if (!delta) return std::make_tuple(outermost, innermost, identity);
    // a second row of determinant 1 under which no distance turns negative (strictly positive where asked)
    auto second_row = [&](int a, int b, bool strictly, int &gamma, int &sigma) {
        for (int size = 0; size <= 2 * LARGEST_COEFFICIENT; size++)
            for (int g = -size; g <= size; g++)
                for (int sg : {size - std::abs(g), -(size - std::abs(g))}) {
                    if (a * sg - b * g != 1 || !none(delta, row(g, sg) + (strictly ? " <= 0" : " < 0"))) continue;
                    gamma = g;
                    sigma = sg;
                    return true;
                }
        return false;
    };
    for (int sign : {1, -1}) {
        int found = 0;
        for (auto &ab : candidates(sign)) {
            const std::string across = row(ab.first, ab.second);
            if (!none(delta, across + " < 0")) continue;
            int gamma, sigma;
            if (none(delta, across + " = 0") && found < nb_parallel && second_row(ab.first, ab.second, false, gamma, sigma)) {
                innermost.push_back(std::make_tuple(ab.first, ab.second, gamma, sigma));
                found++;
            }
            if (none(delta, across + " > 0") && outermost.empty() && second_row(ab.first, ab.second, true, gamma, sigma))
                outermost.push_back(std::make_tuple(ab.first, ab.second, gamma, sigma));
        }
    }
    if (none(delta, "di < 0"))
        for (int gamma = 0; gamma <= LARGEST_COEFFICIENT; gamma++)
            if (none(delta, row(gamma, 1) + " < 0")) {
                identity.push_back(std::make_tuple(1, 0, gamma, 1));
                break;
            }
    isl_set_free(delta);
    return std::make_tuple(outermost, innermost, identity);
}

// ------------------------------------------------------------------ the implicit function

void perform_full_dependency_analysis() { global::get_implicit_function()->perform_full_dependency_analysis(); }
bool check_legality_of_function() { return global::get_implicit_function()->check_legality_for_function(); }
void prepare_schedules_for_legality_checks(bool reset_static_dimesion) {
    global::get_implicit_function()->prepare_schedules_for_legality_checks(reset_static_dimesion);
}
bool loop_parallelization_is_legal(var i, std::vector<computation *> fused_computations) {
    return global::get_implicit_function()->loop_parallelization_is_legal(i, fused_computations);
}
bool loop_unrolling_is_legal(var i, std::vector<computation *> fused_computations) {
    return global::get_implicit_function()->loop_unrolling_is_legal(i, fused_computations);
}
bool loop_vectorization_is_legal(var i, std::vector<computation *> fused_computations) {
    return global::get_implicit_function()->loop_vectorization_is_legal(i, fused_computations);
}

}  // namespace tiramisu
