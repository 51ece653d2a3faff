// HIP back-end driver: walks the lowered loop program, replaces every GPU-tagged loop nest
// by kernel launches, prints the host glue as plain C++ (no HIP headers: it reaches the
// device only through the tiramisu_hip_* C ABI), compiles the kernels to a gfx950 code
// object with hipcc and embeds that object into the host object file.
//
// Artefacts for codegen(..., "f.o", true):
//   f.o.hip       kernel source            (kept when HIP_NO_OVERWRITE is set, like the
//   f.o.hsaco     gfx950 code object        reference's CUDA_NO_OVERWRITE, tiramisu_codegen_cuda.cpp:1808)
//   f.o.host.cpp  host glue source
//   f.o           host object; exports  extern "C" int <function>(halide_buffer_t *...)
#include "hip_backend.h"
#include "kernels/target_gfx950.h"

#include <cstdio>
#include <cstdlib>
#include <fcntl.h>
#include <fstream>
#include <sstream>
#include <sys/wait.h>
#include <unistd.h>

#include "util.h"

namespace tiramisu {
namespace hipgen {

using lir::leaf_kind;
using lir::node;
using lir::node_kind;
using lir::node_ptr;

static int kernel_counter = 0;  // process-wide, like the reference's kernel_count (tiramisu_codegen_cuda.cpp:1320)
int context::next_kernel_id() { return kernel_counter++; }
int context::peek_next_kernel_id() { return kernel_counter; }
void context::set_next_kernel_id(int id) { kernel_counter = id; }

namespace {

bool depends_on(const expr &e, const std::set<std::string> &names) {
    bool d = false;
    e.visit([&](const expr &x) {
        if (x.get_expr_type() == e_var && names.count(x.get_name())) d = true;
    });
    return d;
}

std::string pad(int n) { return std::string(n * 4, ' '); }

// ---------------------------------------------------------------- generic kernel

struct generic_kernel_gen {
    context &ctx;
    function *f;
    c_printer dev;
    std::set<std::string> used_buffers, used_scalars;
    std::set<std::string> inner;        // iterators and let names defined inside the kernel
    std::set<std::string> declared;     // buffers declared by an allocate leaf inside the kernel
    std::vector<expr> grid_ext[3], block_ext[3];
    int loops_per_dim[2][3] = {{0, 0, 0}, {0, 0, 0}};
    std::ostringstream body;

    generic_kernel_gen(context &c) : ctx(c), f(c.f) {
        dev.fct = f;
        dev.device = true;
        dev.used_buffers = &used_buffers;
        dev.used_scalars = &used_scalars;
    }

    std::set<std::string> streamed;      // global buffers that the kernel writes and never reads
    void find_streaming_stores(const node_ptr &root) {
        const char *o = backend_option("TIRAMISU_HIP_STREAMING_STORES");
        if (!o || std::string(o) == "0") return;
        std::set<std::string> written, read;
        lir::walk(root, [&](const node_ptr &n) {
            if (n->kind != node_kind::leaf) return;
            if (n->lhs && n->lhs->get_location() == memory_location::global) written.insert(n->lhs->get_name());
            auto scan = [&](const expr &e) {
                if (e.is_defined()) e.visit([&](const expr &x) { if (x.get_expr_type() == e_op && (x.get_op_type() == o_access || x.get_op_type() == o_address_of || x.get_op_type() == o_buffer)) read.insert(x.get_name()); });
            };
            scan(n->rhs);
            scan(n->predicate);
            for (auto &l : n->lets) scan(l.second);
            for (auto &ix : n->lhs_index) scan(ix);
            if (n->copy_from) read.insert(n->copy_from->get_name());
            if (n->copy_to) read.insert(n->copy_to->get_name());
        });
        for (auto &w : written)
            if (!read.count(w)) streamed.insert(w);
        dev.streaming_stores = &streamed;
    }

    void prepass(const node_ptr &root) {
        find_streaming_stores(root);
        lir::walk(root, [&](const node_ptr &n) {
            if (n->kind == node_kind::loop) {
                inner.insert(n->iterator);
                loops_by_iterator[n->iterator].push_back(n);
                // Statements fused into one nest may disagree about a loop level: a block dimension for those tagged
                // (block, block, thread, thread), a thread dimension for those tagged (block, thread).  The loop can be
                // one thing only: it is a block dimension (which is how it is emitted), and the statements that took
                // it for their thread loop have no thread loop around them any more (they run once per workgroup, below).
                if (n->gpu_block >= 0 && n->gpu_thread >= 0) { n->gpu_thread = -1; conflicting_tags = true; }
                if (n->gpu_block >= 0) loops_per_dim[0][n->gpu_block]++;
                if (n->gpu_thread >= 0) loops_per_dim[1][n->gpu_thread]++;
            }
            if (n->kind == node_kind::leaf) {
                for (auto &l : n->lets) inner.insert(l.first);
                if (n->lkind == leaf_kind::let) inner.insert(n->comp->get_name());
            }
        });
        choose_lane_dimension(root);
        choose_workgroup_shape(root);
        choose_block_order(root);
        if (!backend_option("TIRAMISU_HIP_NO_WAVE_REDUCTION")) {
            std::vector<node_ptr> stack;
            find_reductions(root, stack);
        }
        if (kernel_has_thread_loops()) mark_once_per_workgroup(root);
        check_shared_memory(root);
    }

    // ---- the race check of LDS (option hip_check_shared_memory: "1" stops code generation at a finding, "warn"
    // prints it and goes on).  The reference leaves barriers to the program (tiramisu_codegen_cuda.cpp:1240-1242)
    // and this emitter drops barriers that it takes to be redundant, so the check looks at the kernel as it will be
    // emitted.  Between two barriers every thread of the workgroup may be anywhere, so two accesses of that region
    // to one element of a shared buffer, one of them a write, must come from one thread.  The check finds who
    // touches what by evaluation: for every access it runs through all values of the thread loops and of the serial
    // loops without a barrier around it (their iterations all lie in one region) and notes the thread of each
    // element.  Serial loops with a barrier inside are walked for three consecutive values of their iterator, with
    // what one iteration leaves pending meeting the next; block iterators take their first value (workgroups do not
    // share LDS); conditions and predicates that evaluate to false exclude the access.  An access whose index or
    // loop bounds do not evaluate (a size known only at run time) is reported as not analysed and stops nothing.
    struct shared_access {
        std::string buffer, text, who, key;
        bool write = false, known = true;
        std::map<long, long> owner;       // element -> thread, or -2: several threads
    };
    static bool evaluate(const expr &e, const std::map<std::string, long> &env, long &out) {
        if (!e.is_defined()) return false;
        if (e.get_expr_type() == e_val) {
            if (e.get_data_type() == p_float32 || e.get_data_type() == p_float64) return false;
            out = (long)e.get_int_val();
            return true;
        }
        if (e.get_expr_type() == e_var) {
            auto it = env.find(e.get_name());
            if (it == env.end()) return false;
            out = it->second;
            return true;
        }
        if (e.get_expr_type() != e_op) return false;
        long a = 0, b = 0, c = 0;
        const op_t op = e.get_op_type();
        if (op == o_access || op == o_call || op == o_address_of || op == o_lin_index || op == o_buffer) return false;
        const int n = e.get_n_arg();
        if ((op == o_logical_and || op == o_logical_or) && n == 2) {
            // one side may be known only at run time: false && x is false, true || x is true
            const bool has_a = evaluate(e.get_operand(0), env, a), has_b = evaluate(e.get_operand(1), env, b);
            const long decides = op == o_logical_and ? 0 : 1;
            if ((has_a && (a != 0) == decides) || (has_b && (b != 0) == decides)) { out = decides; return true; }
            if (!has_a || !has_b) return false;
            out = op == o_logical_and ? (a && b) : (a || b);
            return true;
        }
        if (n >= 1 && !evaluate(e.get_operand(0), env, a)) return false;
        if (op == o_select || op == o_cond) {           // only the branch taken must evaluate
            return n == 3 && evaluate(e.get_operand(a ? 1 : 2), env, out);
        }
        if (n >= 2 && !evaluate(e.get_operand(1), env, b)) return false;
        if (n >= 3 && !evaluate(e.get_operand(2), env, c)) return false;
        switch (op) {
        case o_minus: out = -a; return true;
        case o_cast: out = a; return e.get_data_type() != p_float32 && e.get_data_type() != p_float64;
        case o_add: out = a + b; return true;
        case o_sub: out = a - b; return true;
        case o_mul: out = a * b; return true;
        case o_div: if (!b) return false; out = a / b; return true;
        case o_mod: if (!b) return false; out = a % b; return true;
        case o_floordiv: if (!b) return false; out = a / b - ((a % b != 0) && ((a < 0) != (b < 0))); return true;
        case o_floormod: if (!b) return false; out = ((a % b) + b) % b; return true;
        case o_logical_and: out = a && b; return true;
        case o_logical_or: out = a || b; return true;
        case o_logical_not: out = !a; return true;
        case o_eq: out = a == b; return true;
        case o_ne: out = a != b; return true;
        case o_le: out = a <= b; return true;
        case o_lt: out = a < b; return true;
        case o_ge: out = a >= b; return true;
        case o_gt: out = a > b; return true;
        case o_max: out = std::max(a, b); return true;
        case o_min: out = std::min(a, b); return true;
        case o_right_shift: out = a >> b; return true;
        case o_left_shift: out = a << b; return true;
        default: return false;
        }
    }
    // A loop bound for the enumeration: its value, or -- for min(a, b) as an upper bound and max(a, b) as a lower one,
    // the shape of a partial tile's bound -- the side that has a value.  That may run through more iterations than
    // the loop has (threads that a guard keeps out), which can add findings but cannot hide one.
    static bool evaluate_bound(const expr &e, const std::map<std::string, long> &env, bool upper, long &out) {
        if (evaluate(e, env, out)) return true;
        if (!e.is_defined() || e.get_expr_type() != e_op) return false;
        if (e.get_op_type() == o_cast && e.get_n_arg() == 1) return evaluate_bound(e.get_operand(0), env, upper, out);
        if (e.get_op_type() != (upper ? o_min : o_max) || e.get_n_arg() != 2) return false;
        long a = 0, b = 0;
        const bool has_a = evaluate_bound(e.get_operand(0), env, upper, a), has_b = evaluate_bound(e.get_operand(1), env, upper, b);
        if (!has_a && !has_b) return false;
        out = has_a && has_b ? (upper ? std::min(a, b) : std::max(a, b)) : has_a ? a : b;
        return true;
    }
    static bool contains_sync(const node_ptr &n) {
        bool found = false;
        lir::walk(n, [&](const node_ptr &x) { if (is_sync(x)) found = true; });
        return found;
    }
    void check_shared_memory(const node_ptr &root) {
        const char *mode = backend_option("TIRAMISU_HIP_CHECK_SHARED_MEMORY");
        if (!mode || std::string(mode) == "0") return;
        std::vector<shared_access> pending;
        std::vector<std::string> findings, unanalysed;
        std::map<std::string, long> env;                          // iterators with one value at a time
        std::vector<node_ptr> run_through;                        // thread loops and barrier-free serial loops around the statement
        std::vector<std::pair<expr, bool>> conditions;            // conditions around the statement and the truth value that leads to it
        c_printer pr;
        pr.fct = f;
        pr.device = true;
        auto note = [](std::vector<std::string> &list, const std::string &line) {
            if (std::find(list.begin(), list.end(), line) == list.end()) list.push_back(line);
        };
        auto thread_name = [](long t) {
            if (t == -2) return std::string("several threads");
            std::string s;
            for (int d = 2; d >= 0; d--) s += (s.empty() ? "" : ",") + std::to_string((t >> (12 * d)) & 4095);
            return "thread (z,y,x) = (" + s + ")";
        };
        // who touches which element: all values of the loops of run_through, innermost last
        auto owners = [&](shared_access &acc, const buffer *b, const std::vector<expr> &index, const node_ptr &leaf) {
            const expr element = lir::simplify(lir::linearize(b, index));
            long budget = 1L << 22;
            std::map<std::string, long> at = env;
            std::function<void(size_t, long)> level = [&](size_t d, long thread) {
                if (!acc.known) return;
                if (d == run_through.size()) {
                    if (--budget < 0) { acc.known = false; return; }
                    long v = 0;
                    for (auto &c : conditions) {
                        if (!evaluate(c.first, at, v)) continue;                // unknown: taken to hold
                        if ((v != 0) != c.second) return;
                    }
                    for (auto &l : leaf->lets) { if (evaluate(l.second, at, v)) at[l.first] = v; else at.erase(l.first); }
                    if (leaf->predicate.is_defined() && evaluate(leaf->predicate, at, v) && !v) return;
                    if (!evaluate(element, at, v)) { acc.known = false; return; }
                    auto it = acc.owner.find(v);
                    if (it == acc.owner.end()) acc.owner[v] = thread;
                    else if (it->second != thread) it->second = -2;
                    return;
                }
                const node_ptr &l = run_through[d];
                long first = 0, last = 0, step = 1;
                if (!evaluate_bound(l->init, at, false, first) || !evaluate_bound(l->upper, at, true, last) ||
                    (l->increment.is_defined() && !evaluate(l->increment, at, step)) || step <= 0) { acc.known = false; return; }
                for (long v = first; v <= last && acc.known; v += step) {
                    at[l->iterator] = v;
                    level(d + 1, l->gpu_thread >= 0 ? thread | ((v & 4095) << (12 * l->gpu_thread)) : thread);
                }
                at.erase(l->iterator);
            };
            level(0, 0);
        };
        auto meet = [&](shared_access now) {
            for (auto &p : pending) if (p.key == now.key) return;               // has met everything already
            const std::string here = now.who + (now.write ? " writes " : " reads ") + now.buffer + now.text;
            if (!now.known) note(unanalysed, here + ": the index or a loop bound around it has no value at compile time");
            if (now.known && now.write)
                for (auto &o : now.owner)
                    if (o.second == -2) { note(findings, here + ": several threads write element " + std::to_string(o.first)); break; }
            for (auto &p : pending) {
                if (p.buffer != now.buffer || (!p.write && !now.write) || !p.known || !now.known) continue;
                const bool p_smaller = p.owner.size() < now.owner.size();
                const auto &small = p_smaller ? p.owner : now.owner;
                const auto &large = p_smaller ? now.owner : p.owner;
                for (auto &o : small) {
                    auto it = large.find(o.first);
                    if (it == large.end() || (it->second == o.second && o.second != -2)) continue;
                    const long tp = p_smaller ? o.second : it->second, tn = p_smaller ? it->second : o.second;
                    note(findings, "no sync between \"" + p.who + (p.write ? " writes " : " reads ") + p.buffer + p.text + "\" and \"" + here +
                                   "\": element " + std::to_string(o.first) + " is touched by " + thread_name(tp) + " in the first and by " +
                                   thread_name(tn) + " in the second");
                    break;
                }
            }
            pending.push_back(std::move(now));
        };
        auto access = [&](const buffer *b, const std::vector<expr> &index, bool write, const node_ptr &leaf) {
            shared_access acc;
            acc.buffer = b->get_name();
            for (auto &e : index) acc.text += "[" + pr.print(lir::simplify(e)) + "]";
            acc.who = leaf->comp ? leaf->comp->get_name() : std::string("a statement");
            acc.write = write;
            acc.key = acc.who + (write ? " W " : " R ") + acc.buffer + acc.text;
            for (auto &v : env) acc.key += " " + v.first + "=" + std::to_string(v.second);
            for (auto &p : pending) if (p.key == acc.key) return;
            owners(acc, b, index, leaf);
            meet(std::move(acc));
        };
        std::function<void(const node_ptr &)> go = [&](const node_ptr &n) {
            if (!n) return;
            if (once_per_workgroup.count(n.get())) { pending.clear(); return; }     // one thread, a barrier before and after
            switch (n->kind) {
            case node_kind::block:
                for (auto &c : without_redundant_barriers(n->children)) go(c);
                return;
            case node_kind::cond:
                conditions.push_back({n->condition, true});
                go(n->then_body);
                conditions.back().second = false;
                go(n->else_body);
                conditions.pop_back();
                return;
            case node_kind::loop: {
                long first = 0, last = 0, step = 1;
                const bool bounded = evaluate_bound(n->init, env, false, first) && evaluate_bound(n->upper, env, true, last) &&
                                     (!n->increment.is_defined() || evaluate(n->increment, env, step)) && step > 0;
                if (n->gpu_block >= 0) {
                    // the first workgroup stands for all: only the first value is needed, not how many there are
                    if (evaluate_bound(n->init, env, false, first)) env[n->iterator] = first;
                    go(n->body);
                    env.erase(n->iterator);
                } else if (n->gpu_thread >= 0 || !contains_sync(n->body)) {
                    run_through.push_back(n);
                    go(n->body);
                    run_through.pop_back();
                } else {
                    // a barrier inside: one value at a time, what an iteration leaves pending meets the next one
                    for (int k = 0; k < 3; k++) {
                        if (bounded && first + k * step > last) break;
                        if (bounded) env[n->iterator] = first + k * step;
                        go(n->body);
                    }
                    env.erase(n->iterator);
                }
                return;
            }
            case node_kind::leaf: {
                if (n->lkind == leaf_kind::sync) { pending.clear(); return; }
                auto reads = [&](const expr &e) {
                    if (!e.is_defined()) return;
                    e.visit([&](const expr &x) {
                        if (x.get_expr_type() != e_op || x.get_op_type() != o_access) return;
                        auto it = f->get_buffers().find(x.get_name());
                        if (it != f->get_buffers().end() && it->second->get_location() == memory_location::shared)
                            access(it->second, x.get_access(), false, n);
                    });
                };
                reads(n->rhs);
                reads(n->predicate);
                for (auto &l : n->lets) reads(l.second);
                for (auto &ix : n->lhs_index) reads(ix);
                if (n->lhs && n->lhs->get_location() == memory_location::shared) access(n->lhs, n->lhs_index, true, n);
                return;
            }
            }
        };
        go(root);
        for (auto &l : unanalysed) std::cerr << "LDS race check, not analysed: " << l << std::endl;
        for (auto &l : findings) std::cerr << "LDS race check: " << l << std::endl;
        if (!findings.empty() && std::string(mode) != "warn") ERROR("shared-memory accesses of different threads are not separated by a sync", true);
    }

    // ---- which thread-mapped loop runs along the lanes.  The front-end numbers the tagged thread levels from
    // the innermost outwards (x, y, z: tiramisu_codegen_cuda.cpp:560-617), whatever the accesses look like: a
    // program that tiles (i, j) with i the contiguous index of its buffers -- the image pipelines of
    // benchmarks/halide all do -- gets threadIdx.x on the strided index, and the 64 lanes of a wavefront touch 16
    // rows.  Which hardware index carries which tagged loop is not part of the program's meaning (the threads of
    // a block are unordered), so the kernel may renumber: the dimension in which most accesses to memory have
    // unit stride becomes x.  Not done when some statement stores to memory at an element that does not involve
    // every thread loop around it (a sum or a broadcast across threads: the lowering of those is tied to x).
    void choose_lane_dimension(const node_ptr &root) {
        if (backend_option("TIRAMISU_HIP_KEEP_THREAD_DIMENSIONS")) return;
        int used = 0;
        for (int d = 0; d < 3; d++) used += loops_per_dim[1][d] > 0;
        if (used < 2) return;
        long score[3] = {0, 0, 0};
        bool veto = false;
        std::vector<node_ptr> stack;
        std::function<void(const node_ptr &)> go = [&](const node_ptr &n) {
            if (!n || veto) return;
            if (n->kind == node_kind::loop) stack.push_back(n);
            if (n->kind == node_kind::leaf) {
                std::string it[3];
                for (auto &l : stack)
                    if (l->gpu_thread >= 0) it[l->gpu_thread] = l->iterator;
                auto count = [&](const buffer *b, const std::vector<expr> &index) {
                    if (!b || index.size() != b->get_dim_sizes().size()) return;
                    if (b->get_location() != memory_location::global && b->get_location() != memory_location::host &&
                        b->get_location() != memory_location::shared) return;
                    const expr lin = lir::simplify(lir::linearize(b, index));
                    for (int d = 0; d < 3; d++) {
                        if (it[d].empty() || !lir::mentions(lin, it[d])) continue;
                        bool ok = true;
                        const expr c = lir::simplify(lir::coefficient(lin, it[d], ok));
                        // a strided access to global memory is one transaction per lane, a strided LDS access a few
                        // conflict cycles: global accesses decide, LDS accesses break ties
                        if (ok && c.is_integer_literal() && (c.get_int_val() == 1 || c.get_int_val() == -1))
                            score[d] += b->get_location() == memory_location::shared ? 1 : 16;
                    }
                };
                auto count_loads = [&](const expr &e) {
                    if (!e.is_defined()) return;
                    e.visit([&](const expr &x) {
                        if (x.get_expr_type() != e_op || x.get_op_type() != o_access) return;
                        auto b = f->get_buffers().find(x.get_name());
                        if (b != f->get_buffers().end()) count(b->second, x.get_access());
                    });
                };
                if (n->lkind == leaf_kind::assign && n->lhs) {
                    const memory_location where = n->lhs->get_location();
                    if (where == memory_location::global || where == memory_location::host || where == memory_location::shared)
                        for (int d = 0; d < 3; d++) {
                            if (it[d].empty() && loops_per_dim[1][d] > 0) veto = true;    // outside that dimension's thread loops: runs once per workgroup (below)
                            if (it[d].empty()) continue;
                            bool involved = false;
                            for (auto &e : n->lhs_index) involved = involved || lir::mentions(e, it[d]);
                            if (!involved) veto = true;
                        }
                    count(n->lhs, n->lhs_index);
                }
                if (n->lkind == leaf_kind::assign || n->lkind == leaf_kind::let) {
                    count_loads(n->rhs);
                    count_loads(n->predicate);
                    for (auto &l : n->lets) count_loads(l.second);
                }
                if (n->lkind == leaf_kind::call) veto = true;
            }
            for (auto &c : n->children) go(c);
            go(n->body);
            go(n->then_body);
            go(n->else_body);
            if (n->kind == node_kind::loop) stack.pop_back();
        };
        go(root);
        threads_independent = !veto;
        if (veto) return;
        int best = 0;
        for (int d = 1; d < 3; d++)
            if (loops_per_dim[1][d] > 0 && score[d] > score[best]) best = d;
        if (best == 0) return;
        if (best == 2) {
            // what x carried moves to z, and a workgroup is at most 64 deep along z
            bool fits = true;
            lir::walk(root, [&](const node_ptr &n) {
                if (n->kind != node_kind::loop || n->gpu_thread != 0) return;
                bool guard;
                expr first;
                const expr ext = lir::simplify(host_extent(n, first, guard));
                if (!ext.is_integer_literal() || ext.get_int_val() > 64) fits = false;
            });
            if (!fits) return;
        }
        lir::walk(root, [&](const node_ptr &n) {
            if (n->kind != node_kind::loop) return;
            if (n->gpu_thread == 0) n->gpu_thread = best;
            else if (n->gpu_thread == best) n->gpu_thread = 0;
        });
        std::swap(loops_per_dim[1][0], loops_per_dim[1][best]);
        lanes_renumbered = true;
    }
    bool lanes_renumbered = false;
    bool threads_independent = false;   // every store to memory involves every thread loop around it, no calls

    // ---- how wide a workgroup is.  A program tiled gpu_tile(i, j, 16, 16) gives a wavefront a patch of 16 x 4
    // points: four short row segments per access.  Where the points of a kernel have nothing to do with one
    // another (no LDS, no barrier, no sum across threads) the grouping of points into workgroups is free as well,
    // so such a kernel with a two-dimensional grid and block deals its points out again: along x a workgroup is
    // 64 wide (one wavefront = 64 consecutive points of a row), along y as high as keeps its thread count, and
    // every thread recovers the block and thread iterators of the point it stands for,
    //     g = 64 * blockIdx.x + threadIdx.x,  block iterator = g / S,  thread iterator = g % S,
    // S being the program's tile extent; the program's own guards, written in those iterators, stay as they are.
    struct retiling {
        bool on = false;
        const node *block[2] = {nullptr, nullptr}, *thread[2] = {nullptr, nullptr};
        long tile[2] = {0, 0}, wide[2] = {0, 0};     // the program's thread extents, the workgroup's
    } retile;
    void choose_workgroup_shape(const node_ptr &root) {
        if (backend_option("TIRAMISU_HIP_KEEP_TILES") || !threads_independent) return;
        for (int d = 0; d < 3; d++)
            if (loops_per_dim[0][d] != (d < 2) || loops_per_dim[1][d] != (d < 2)) return;
        bool plain = true;
        node_ptr block[2], thread[2];
        std::vector<node_ptr> order;      // mapped loops from the outermost inwards
        lir::walk(root, [&](const node_ptr &n) {
            if (n->kind == node_kind::leaf) {
                if (n->lkind == leaf_kind::sync || n->lkind == leaf_kind::call || n->lkind == leaf_kind::copy) plain = false;
                if ((n->lkind == leaf_kind::allocate || n->lkind == leaf_kind::release) && n->target &&
                    n->target->get_location() == memory_location::shared) plain = false;
                auto shared = [&](const expr &e) {
                    if (!e.is_defined()) return;
                    e.visit([&](const expr &x) {
                        if (x.get_expr_type() != e_op || x.get_op_type() != o_access) return;
                        auto b = f->get_buffers().find(x.get_name());
                        if (b != f->get_buffers().end() && b->second->get_location() == memory_location::shared) plain = false;
                    });
                };
                if (n->lhs && n->lhs->get_location() == memory_location::shared) plain = false;
                shared(n->rhs);
                shared(n->predicate);
                for (auto &l : n->lets) shared(l.second);
            }
            if (n->kind != node_kind::loop) return;
            if (n->gpu_block >= 0) { block[n->gpu_block] = n; order.push_back(n); }
            if (n->gpu_thread >= 0) { thread[n->gpu_thread] = n; order.push_back(n); }
        });
        if (!plain || order.size() != 4 || order[0]->gpu_block < 0 || order[1]->gpu_block < 0) return;
        // the four mapped loops sit directly inside one another (a thread may then define all four iterators at once)
        if (order[0] != root) return;
        for (int i = 0; i + 1 < 4; i++) {
            node_ptr inside = order[i]->body;
            while (inside && inside->kind == node_kind::block && inside->children.size() == 1) inside = inside->children[0];
            if (inside != order[i + 1]) return;
        }
        long S[2];
        for (int d = 0; d < 2; d++) {
            bool guard;
            expr first;
            const expr ext = lir::simplify(host_extent(thread[d], first, guard));
            if (!ext.is_integer_literal() || !lir::simplify(thread[d]->init).is_integer_literal() || lir::simplify(thread[d]->init).get_int_val() != 0) return;
            if (!lir::simplify(block[d]->init).is_integer_literal() || lir::simplify(block[d]->init).get_int_val() != 0) return;
            if (depends_on(block[d]->upper, inner)) return;
            S[d] = ext.get_int_val();
            if (S[d] < 1 || (S[d] & (S[d] - 1)) != 0) return;
        }
        const long W = ttarget::WAVEFRONT;
        if (S[0] >= W || (S[0] * S[1]) % W != 0) return;
        // the block loop that tiles the same index as the thread loop on x: its coefficient in some access to
        // global memory is the tile extent times the thread iterator's
        int partner = -1;
        lir::walk(root, [&](const node_ptr &n) {
            if (n->kind != node_kind::leaf || partner >= 0) return;
            auto look = [&](const buffer *b, const std::vector<expr> &index) {
                if (partner >= 0 || !b || index.size() != b->get_dim_sizes().size() || b->get_location() != memory_location::global) return;
                const expr lin = lir::simplify(lir::linearize(b, index));
                bool ok = true;
                const expr ct = lir::simplify(lir::coefficient(lin, thread[0]->iterator, ok));
                if (!ok || !ct.is_integer_literal() || ct.get_int_val() == 0) return;
                for (int d = 0; d < 2; d++) {
                    bool okb = true;
                    const expr cb = lir::simplify(lir::coefficient(lin, block[d]->iterator, okb));
                    if (okb && cb.is_integer_literal() && cb.get_int_val() == ct.get_int_val() * S[0]) partner = d;
                }
            };
            if (n->lkind == leaf_kind::assign && n->lhs) look(n->lhs, n->lhs_index);
            if (n->rhs.is_defined())
                n->rhs.visit([&](const expr &x) {
                    if (x.get_expr_type() != e_op || x.get_op_type() != o_access) return;
                    auto b = f->get_buffers().find(x.get_name());
                    if (b != f->get_buffers().end()) look(b->second, x.get_access());
                });
        });
        if (partner < 0) return;
        if (partner == 1) {
            std::swap(block[0], block[1]);
            block[0]->gpu_block = 0;
            block[1]->gpu_block = 1;
        }
        retile.on = true;
        for (int d = 0; d < 2; d++) {
            retile.block[d] = block[d].get();
            retile.thread[d] = thread[d].get();
            retile.tile[d] = S[d];
        }
        retile.wide[0] = W;
        retile.wide[1] = S[0] * S[1] / W;
    }

    // ---- which tile a workgroup takes.  Workgroups are dealt round-robin to the chip's XCDs, each with an L2 of
    // its own, in the order x fastest: neighbouring tiles of a 2-D grid run on different XCDs, and a cache line
    // that several tiles touch (16 one-byte pixels of a 128-byte line per tile in the reference's image pipelines;
    // the halo of a stencil tile) is fetched from memory once per XCD.  Workgroups being unordered, a kernel with
    // a two-dimensional grid renumbers them: XCD c takes the c-th eighth of the tiles, walked with the block
    // dimension fastest whose iterator has the smallest stride in the accesses to global memory, so that tiles
    // that share lines meet in one L2 at about the same time.  Done only where tiles share data -- a tile is at
    // most 32 bytes wide along that dimension (four tiles or more per line), the kernel stages data in LDS (halos,
    // operand panels), or some access to global memory does not depend on one of the two block iterators (a panel
    // that a row of tiles re-reads): for a plain streaming kernel with wide tiles the renumbering only costs its
    // integer division per workgroup (the 8192 x 8192 copy kernel, one element per thread: 0.152 ms against 0.105).
    int fast_block_dim = -1;      // 0 or 1 when the workgroups are renumbered
    void choose_block_order(const node_ptr &root) {
        if (backend_option("TIRAMISU_HIP_KEEP_BLOCK_ORDER")) return;
        if (loops_per_dim[0][0] != 1 || loops_per_dim[0][1] != 1 || loops_per_dim[0][2] != 0) return;
        std::string it[2];
        lir::walk(root, [&](const node_ptr &n) {
            if (n->kind == node_kind::loop && n->gpu_block >= 0 && n->gpu_block < 2) it[n->gpu_block] = n->iterator;
        });
        long stride[2] = {0, 0};      // smallest literal |coefficient| x element size of the block iterator over the global accesses
        bool other[2] = {false, false};   // ... or some access in which it has a non-literal coefficient
        bool shares = false;              // tiles share data (LDS staging, or an access that ignores a block iterator)
        auto count = [&](const buffer *b, const std::vector<expr> &index) {
            if (!b || index.size() != b->get_dim_sizes().size()) return;
            if (b->get_location() == memory_location::shared) shares = true;
            if (b->get_location() != memory_location::global && b->get_location() != memory_location::host) return;
            const expr lin = lir::simplify(lir::linearize(b, index));
            const long bytes = (long)primitive_size(b->get_elements_type());
            for (int d = 0; d < 2; d++) {
                if (!lir::mentions(lin, it[d])) { shares = true; continue; }
                bool ok = true;
                const expr c = lir::simplify(lir::coefficient(lin, it[d], ok));
                if (ok && c.is_integer_literal() && c.get_int_val() != 0) {
                    const long a = std::labs(c.get_int_val()) * bytes;
                    stride[d] = stride[d] == 0 ? a : std::min(stride[d], a);
                } else {
                    other[d] = true;
                }
            }
        };
        lir::walk(root, [&](const node_ptr &n) {
            if (n->kind != node_kind::leaf) return;
            if (n->lkind == leaf_kind::assign && n->lhs) count(n->lhs, n->lhs_index);
            auto loads = [&](const expr &e) {
                if (!e.is_defined()) return;
                e.visit([&](const expr &x) {
                    if (x.get_expr_type() != e_op || x.get_op_type() != o_access) return;
                    auto b = f->get_buffers().find(x.get_name());
                    if (b != f->get_buffers().end()) count(b->second, x.get_access());
                });
            };
            if (n->lkind == leaf_kind::assign || n->lkind == leaf_kind::let) {
                loads(n->rhs);
                loads(n->predicate);
                for (auto &l : n->lets) loads(l.second);
            }
        });
        // one dimension with a literal stride, smaller than the other's or the other's symbolic (a row pitch)
        if (stride[0] > 0 && (stride[1] == 0 ? other[1] : stride[0] < stride[1])) fast_block_dim = 0;
        else if (stride[1] > 0 && (stride[0] == 0 ? other[0] : stride[1] < stride[0])) fast_block_dim = 1;
        if (fast_block_dim >= 0 && !shares && stride[fast_block_dim] > 32) fast_block_dim = -1;
    }

    // ---- sums across threads.  A statement  X[e] = X[e] + term  under a loop mapped to threadIdx.x whose
    // iterator the element e does not involve asks every thread of that loop to add into one element:
    // as written that is a race (the reference emits it as such).  Floating-point addition being what
    // the program asks to be reassociated here, the loop is lowered to a private partial sum per thread,
    // a sum across the lanes of the wavefront with DPP row shifts and broadcasts (across wavefronts
    // through LDS when the loop is wider than a wavefront), and one read-modify-write of X[e] by the last
    // thread of the loop.
    struct thread_reduction { node_ptr leaf; expr term; int width; bool widened; primitive_t type, element_type; op_t op; };   // widened: width exceeds the loop's extent; type: of the partial sums; op: o_add, o_max or o_min
    std::map<const node *, thread_reduction> reductions;   // keyed by the threadIdx.x loop
    int reduction_count = 0;
    std::vector<expr> conds_above;     // conditions between the kernel's root and the node that find_reductions is visiting

    static bool is_same_element(const expr &e, const buffer *b, const std::vector<expr> &idx) {
        if (e.get_expr_type() != e_op || e.get_op_type() != o_access || e.get_name() != b->get_name() || e.get_access().size() != idx.size())
            return false;
        for (size_t i = 0; i < idx.size(); i++)
            if (!lir::simplify(e.get_access()[i]).is_equal(lir::simplify(idx[i]))) return false;
        return true;
    }

    void find_reductions(const node_ptr &n, std::vector<node_ptr> &stack) {
        if (!n) return;
        if (n->kind == node_kind::loop) stack.push_back(n);
        if (n->kind == node_kind::leaf && n->lkind == leaf_kind::assign && n->lhs &&
            n->rhs.is_defined() && n->rhs.get_expr_type() == e_op &&
            (n->rhs.get_op_type() == o_add || n->rhs.get_op_type() == o_max || n->rhs.get_op_type() == o_min))
            consider_reduction(n, stack, !n->predicate.is_defined() && n->lets.empty());
        if (n->kind == node_kind::leaf && n->lkind == leaf_kind::assign && n->lhs && n->rhs.is_defined()) repeated_along_a_thread_dimension(n, stack);
        for (auto &c : n->children) find_reductions(c, stack);
        find_reductions(n->body, stack);
        if (n->kind == node_kind::cond) conds_above.push_back(n->condition);
        find_reductions(n->then_body, stack);
        find_reductions(n->else_body, stack);
        if (n->kind == node_kind::cond) conds_above.pop_back();
        if (n->kind == node_kind::loop) stack.pop_back();
    }

    // An update of an element from its own value (x = x + ..., x = f(x)) that lies inside the thread loops of some of
    // the kernel's thread dimensions but not of all: the threads along the missing dimensions all execute it, so it is
    // applied that many times (a plain store of one value is merely repeated).  The reference emits the same
    // (tiramisu_codegen_cuda.cpp:549-707); say so.  Statements outside all thread loops run on one thread instead.
    void repeated_along_a_thread_dimension(const node_ptr &leaf, const std::vector<node_ptr> &stack) {
        const memory_location where = leaf->lhs->get_location();
        if (where != memory_location::global && where != memory_location::shared) return;
        int inside = 0, used = 0;
        for (auto &l : stack) if (l->gpu_thread >= 0) inside |= 1 << l->gpu_thread;
        for (int d = 0; d < 3; d++) if (loops_per_dim[1][d] > 0) used |= 1 << d;
        if (inside == 0 || inside == used) return;
        bool reads_itself = false;
        leaf->rhs.visit([&](const expr &x) { if (is_same_element(x, leaf->lhs, leaf->lhs_index)) reads_itself = true; });
        if (!reads_itself) return;
        std::string missing;
        for (int d = 0; d < 3; d++) if ((used & ~inside) & (1 << d)) missing += std::string(missing.empty() ? "" : ", ") + "xyz"[d];
        std::cerr << "GPU mapping: " << leaf->comp->get_name() << " of " << f->get_name() << " updates " << leaf->lhs->get_name()
                  << " from its own value inside some of the kernel's thread loops only: every thread along dimension " << missing
                  << " repeats the update" << std::endl;
    }

    void consider_reduction(const node_ptr &leaf, const std::vector<node_ptr> &stack, bool plain_statement) {
        // registers and thread-local arrays are a thread's own: nothing is shared, whatever the index says
        const memory_location where = leaf->lhs->get_location();
        if (where != memory_location::global && where != memory_location::shared) return;
        expr term;
        if (is_same_element(leaf->rhs.get_operand(0), leaf->lhs, leaf->lhs_index)) term = leaf->rhs.get_operand(1);
        else if (is_same_element(leaf->rhs.get_operand(1), leaf->lhs, leaf->lhs_index)) term = leaf->rhs.get_operand(0);
        else return;
        bool reads_self = false;
        term.visit([&](const expr &x) {
            if (x.get_expr_type() == e_op && x.get_op_type() == o_access && x.get_name() == leaf->lhs->get_name()) reads_self = true;
        });
        if (reads_self) return;
        auto element_involves = [&](const std::string &it) {
            for (auto &e : leaf->lhs_index) if (lir::mentions(e, it)) return true;
            return false;
        };
        // the thread-mapped loops around the statement that its element does not involve
        node_ptr R;
        size_t at = 0;
        bool not_one_loop_on_x = false;     // the lowering takes one loop, on threadIdx.x (consecutive lanes)
        for (size_t d = 0; d < stack.size(); d++)
            if (stack[d]->gpu_thread >= 0 && !element_involves(stack[d]->iterator)) {
                if (R || stack[d]->gpu_thread != 0) not_one_loop_on_x = true;
                if (!R) {
                    R = stack[d];
                    at = d;
                }
            }
        if (!R) return;
        // From here on the statement is known to be a sum that all threads of loop R add to one element.  Where it
        // is not lowered it is emitted as scheduled, like the reference does (tiramisu_codegen_cuda.cpp:549-707):
        // the threads race and the result is wrong, so say so.
        auto left_as_scheduled = [&](const std::string &why) {
            std::cerr << "GPU mapping: the " << (leaf->rhs.get_op_type() == o_add ? "sum " : leaf->rhs.get_op_type() == o_max ? "maximum " : "minimum ") << leaf->comp->get_name() << " over thread loop " << R->iterator << " of " << f->get_name()
                      << " is emitted as scheduled, its threads race on " << leaf->lhs->get_name() << " (" << why << ")" << std::endl;
        };
        if (not_one_loop_on_x) return left_as_scheduled("it runs over several thread loops, or over one that is not on threadIdx.x");
        if (!plain_statement) return left_as_scheduled("the statement carries a predicate or scalar definitions");
        const primitive_t type = leaf->rhs.get_data_type();
        // 8- and 16-bit integers wrap, and the wrap commutes with addition: their partial sums are kept in 32 bits and the
        // final store truncates
        primitive_t partial_type = type;
        const op_t op = leaf->rhs.get_op_type();
        if (op == o_add) {
            if (type == p_int8 || type == p_int16 || type == p_uint8 || type == p_uint16) partial_type = p_uint32;   // unsigned: wraps, never overflows
        } else {
            // a maximum or minimum: widening keeps the order
            if (type == p_int8 || type == p_int16) partial_type = p_int32;
            else if (type == p_uint8 || type == p_uint16) partial_type = p_uint32;
        }
        if (primitive_size(partial_type) != 4 && primitive_size(partial_type) != 8)
            return left_as_scheduled("sums of " + primitive_c_name(type) + " are not lowered: those of integers, float and double are");
        if (loops_per_dim[1][0] != 1) return left_as_scheduled("another loop of the kernel is mapped to threadIdx.x as well");
        // inside it: this statement only, under serial loops whose iterators the element does not involve either
        for (size_t d = at + 1; d < stack.size(); d++)
            if (stack[d]->gpu_thread >= 0 || stack[d]->gpu_block >= 0 || element_involves(stack[d]->iterator))
                return left_as_scheduled("a loop inside the thread loop is mapped too, or selects the element");
        int leaves_inside = 0;
        lir::walk(R, [&](const node_ptr &x) { if (x->kind == node_kind::leaf) leaves_inside++; });
        if (leaves_inside != 1) return left_as_scheduled("the thread loop holds other statements");
        // width of the loop = blockDim.x: a power of two up to a wavefront, or whole wavefronts; an extent in between
        // is rounded up (the lanes beyond the loop's last iteration are masked by the loop's guard and add zero)
        bool guard;
        expr first;
        const expr ext = lir::simplify(host_extent(R, first, guard));
        if (!ext.is_integer_literal()) return left_as_scheduled("the extent of the thread loop is not a constant");
        const long extent = ext.get_int_val();
        if (extent < 2 || extent > 1024) return left_as_scheduled("the extent of the thread loop is " + std::to_string(extent));
        long w = extent;
        if (w <= 64) while (w & (w - 1)) w++;
        else w = (w + 63) / 64 * 64;
        long other_threads = 1;
        for (size_t d = 0; d < at; d++)
            if (stack[d]->gpu_thread >= 0) {
                bool g;
                expr f0;
                const expr e = lir::simplify(host_extent(stack[d], f0, g));
                if (e.is_integer_literal()) other_threads *= e.get_int_val();
            }
        if (w != extent && w * other_threads > 1024)
            return left_as_scheduled("rounded up to " + std::to_string(w) + " lanes the workgroup would exceed 1024 threads");
        const bool waves = w > 64;
        if (waves) {
            // the barrier of the LDS stage must be reached by every thread: no guarded mapped loop around it,
            // no serial loop and no condition (a separated remainder, a hoisted predicate: it may depend on a
            // thread iterator) between the kernel entry and the loop.  (Adding the wavefronts' totals with
            // atomics instead would need no barrier, but nothing would then order them after an initialisation of
            // the element that other wavefronts of the workgroup execute: the barrier is what does that.)
            // a condition on block iterators and kernel parameters alone is the same for the whole workgroup
            std::set<std::string> varies = inner;
            for (size_t d = 0; d < at; d++) if (stack[d]->gpu_block >= 0) varies.erase(stack[d]->iterator);
            for (auto &c : conds_above)
                if (depends_on(c, varies))
                    return left_as_scheduled("wider than a wavefront and under a condition that may differ between threads: the barrier of the sum across wavefronts would not be reached by every thread");
            std::vector<const node *> guarded;
            for (size_t d = 0; d < at; d++) {
                bool g;
                expr f0;
                if (stack[d]->gpu_thread < 0 && stack[d]->gpu_block < 0)
                    return left_as_scheduled("wider than a wavefront and inside a serial loop");
                host_extent(stack[d], f0, g);
                if (stack[d]->gpu_block >= 0) {
                    // the guard of a block loop is the same for the whole workgroup, unless a thread loop lies outside it
                    for (size_t o = 0; o < d; o++)
                        if (stack[o]->gpu_thread >= 0) return left_as_scheduled("wider than a wavefront and inside a block loop that a thread loop encloses");
                    continue;
                }
                if (!g && loops_per_dim[1][stack[d]->gpu_thread] <= 1) continue;
                // A thread loop with a partial last tile: its threads beyond the tile must still reach the barrier.  The
                // loop is emitted with a predicate instead of a branch (live_predicates); that cannot hold statements
                // that declare something for later ones, or a barrier of the program's own.
                bool plain = true;
                lir::walk(stack[d]->body, [&](const node_ptr &x) {
                    if (x->kind == node_kind::cond) plain = false;
                    if (x->kind == node_kind::leaf && (x->lkind != leaf_kind::assign || !x->lhs)) plain = false;
                });
                if (!plain)
                    return left_as_scheduled("wider than a wavefront and inside a mapped loop with a partial last tile that also holds declarations, barriers or conditions");
                guarded.push_back(stack[d].get());
            }
            for (auto g : guarded) predicated_loops.insert(g);
        }
        reductions[R.get()] = {leaf, term, (int)w, w != extent, partial_type, type, op};
    }

    // Thread loops with a partial last tile around a sum across wavefronts: the threads beyond the tile do not branch
    // around the loop's body but carry a predicate (_live_<iterator>), under which the ordinary statements run; the sum
    // itself runs for all of them, the dead ones adding zero and skipping the store.
    std::set<const node *> predicated_loops;
    std::vector<std::string> live_predicates;
    std::string all_live() const {
        std::string c;
        for (auto &p : live_predicates) c += (c.empty() ? "" : " && ") + p;
        return c;
    }
    bool holds_wide_reduction(const node_ptr &n) const {
        bool found = false;
        lir::walk(n, [&](const node_ptr &x) {
            auto r = reductions.find(x.get());
            if (r != reductions.end() && r->second.width > 64) found = true;
        });
        return found;
    }
    void emit_predicated(const node_ptr &n, int ind) {
        if (!n) return;
        if (n->kind == node_kind::block) {
            for (auto &c : n->children) emit_predicated(c, ind);
            return;
        }
        if (n->kind == node_kind::loop && holds_wide_reduction(n)) {
            emit_loop(n, ind);
            return;
        }
        body << pad(ind) << "if (" << all_live() << ") {\n";
        emit(n, ind + 1);
        body << pad(ind) << "}\n";
    }

    void emit_thread_reduction(const node_ptr &n, const thread_reduction &r, int ind) {
        bool guard;
        expr first;
        const expr extent = host_extent(n, first, guard);
        block_ext[0].push_back(r.widened ? expr((int32_t)r.width) : extent);
        if (r.widened) guard = true;
        const std::string acc = "_partial" + std::to_string(reduction_count++);
        body << pad(ind) << "{\n";
        const std::string ctype = primitive_c_name(r.type);
        const std::string opname = r.op == o_max ? "twave::max_op" : r.op == o_min ? "twave::min_op" : "";
        auto combine = [&](const std::string &a, const std::string &b) {
            return r.op == o_add ? a + " + " + b : std::string(r.op == o_max ? "t_max" : "t_min") + "((" + ctype + ")(" + a + "), (" + ctype + ")(" + b + "))";
        };
        body << pad(ind + 1) << ctype << " " << acc << " = " << (r.op == o_add ? "0" : opname + "::identity<" + ctype + ">()")
             << ";   // this thread's share of the " << (r.op == o_add ? "sum" : r.op == o_max ? "maximum" : "minimum") << "\n";
        body << pad(ind + 1) << "{\n";
        body << pad(ind + 2) << "const int32_t " << n->iterator << " = (int32_t)threadIdx.x + " << dev.print(first) << ";\n";
        const std::string live = all_live();
        if (!live.empty() && !guard) {
            guard = true;
            body << pad(ind + 2) << "if (" << live << ") {\n";
        } else if (guard) {
            body << pad(ind + 2) << "if (" << (live.empty() ? "" : live + " && ") << n->iterator << " >= " << dev.print(n->init) << " && " << n->iterator << " <= " << dev.print(n->upper) << ") {\n";
        }
        pending_partial = acc;
        pending_leaf = r.leaf.get();
        pending_term = r.term;
        pending_combine = combine;
        emit(n->body, ind + (guard ? 3 : 2));
        pending_leaf = nullptr;
        if (guard) body << pad(ind + 2) << "}\n";
        body << pad(ind + 1) << "}\n";
        if (r.width <= 64) {
            if (r.op == o_add) body << pad(ind + 1) << acc << " = twave::wave_group_sum<" << r.width << ">(" << acc << ");\n";
            else body << pad(ind + 1) << acc << " = twave::wave_group_reduce<" << r.width << ", " << opname << ">(" << acc << ");\n";
        } else {
            needs_reduction_scratch = true;
            if (primitive_size(r.type) == 8) wide_reduction_scratch = true;
            body << pad(ind + 1) << acc << " = twave::" << (r.op == o_add ? "block_group_sum<" + std::to_string(r.width) : "block_group_reduce<" + std::to_string(r.width) + ", " + opname) << ">(" << acc << ", " << "(" << ctype << " *)_reduction_scratch, "
                 << "(int)(threadIdx.x + blockDim.x * (threadIdx.y + blockDim.y * threadIdx.z)));\n";
        }
        body << pad(ind + 1) << "if (threadIdx.x == " << r.width - 1 << (live.empty() ? "" : " && " + live) << ") "
             << dev.store(r.leaf->lhs, r.leaf->lhs_index, combine(dev.element(r.leaf->lhs, r.leaf->lhs_index), acc), r.op == o_add ? r.element_type : r.type) << "\n";
        body << pad(ind) << "}\n";
        add_include_once(ctx, "#include \"wave_reduce.hip.h\"");
        wave_reductions++;
    }
    std::function<std::string(const std::string &, const std::string &)> pending_combine;
    std::string pending_partial;
    const node *pending_leaf = nullptr;
    expr pending_term;
    bool needs_reduction_scratch = false, wide_reduction_scratch = false;     // wide: a 64-bit sum uses it
    int wave_reductions = 0;

    // Kernel-invariant part of a bound that is a min() (upper bounds) or max() (lower bounds) of
    // several expressions: the arguments that do not involve in-kernel iterators.
    expr invariant_part(const expr &bound, op_t combiner, const std::string &what) {
        std::vector<expr> parts;
        std::function<void(const expr &)> split = [&](const expr &e) {
            if (e.get_expr_type() == e_op && e.get_op_type() == combiner) {
                split(e.get_operand(0));
                split(e.get_operand(1));
            } else if (!depends_on(e, inner)) {
                parts.push_back(e);
            }
        };
        split(bound);
        if (parts.empty()) {
            // every argument varies inside the kernel (a triangular domain: the bound of one mapped loop is a function
            // of another's iterator): the launch covers what the bound can reach over the ranges of those iterators
            expr r;
            if (!over_the_ranges(bound, combiner == o_min, r)) ERROR("GPU-mapped loop " + what + " has no kernel-invariant bound", true);
            return lir::simplify(r);
        }
        expr r = parts[0];
        for (size_t i = 1; i < parts.size(); i++) r = expr(combiner, r, parts[i]);
        return r;
    }

    // A kernel-invariant upper (or lower) bound of an expression of in-kernel loop iterators: each iterator ranges
    // over what the host sees of its loop, sums, differences, products with and quotients by literals and min / max
    // are followed; false for anything else.
    std::map<std::string, std::vector<node_ptr>> loops_by_iterator;
    bool over_the_ranges(const expr &e, bool upper, expr &out) {
        if (!depends_on(e, inner)) { out = e; return true; }
        if (e.get_expr_type() == e_var) {
            auto it = loops_by_iterator.find(e.get_name());
            if (it == loops_by_iterator.end()) return false;
            bool have = false;
            for (auto &n : it->second) {
                expr first; bool guard;
                const expr ext = host_extent(n, first, guard);
                const expr v = upper ? lir::simplify(first + ext - 1) : first;
                out = have ? expr(upper ? o_max : o_min, out, v) : v;
                have = true;
            }
            return have;
        }
        if (e.get_expr_type() != e_op) return false;
        auto literal = [](const expr &x, int64_t &v) {
            const expr c = lir::simplify(x);
            if (!c.is_integer_literal()) return false;
            v = c.get_int_val();
            return true;
        };
        expr a, b;
        int64_t c;
        switch (e.get_op_type()) {
        case o_add:
            if (!over_the_ranges(e.get_operand(0), upper, a) || !over_the_ranges(e.get_operand(1), upper, b)) return false;
            out = a + b; return true;
        case o_sub:
            if (!over_the_ranges(e.get_operand(0), upper, a) || !over_the_ranges(e.get_operand(1), !upper, b)) return false;
            out = a - b; return true;
        case o_mul:
            for (int side = 0; side < 2; side++)
                if (literal(e.get_operand(side), c)) {
                    if (!over_the_ranges(e.get_operand(1 - side), c >= 0 ? upper : !upper, a)) return false;
                    out = e.get_operand(side) * a; return true;
                }
            return false;
        case o_div: case o_floordiv:
            if (!literal(e.get_operand(1), c) || c <= 0 || !over_the_ranges(e.get_operand(0), upper, a)) return false;
            out = expr(e.get_op_type(), a, e.get_operand(1)); return true;
        case o_min: case o_max:
            if (!over_the_ranges(e.get_operand(0), upper, a) || !over_the_ranges(e.get_operand(1), upper, b)) return false;
            out = expr(e.get_op_type(), a, b); return true;
        case o_cast:
            if (!over_the_ranges(e.get_operand(0), upper, a)) return false;
            out = cast(e.get_data_type(), a); return true;
        default: return false;
        }
    }

    // Extent and first value of a mapped loop as seen from the host.  Bounds that vary inside the
    // kernel (partial tiles: min()/max() with outer mapped iterators) contribute their invariant
    // arguments to the launch size and are enforced by a guard in the kernel.  (The reference
    // ignores lower bounds here, tiramisu_codegen_cuda.cpp:523-554.)
    expr host_extent(const node_ptr &n, expr &first, bool &needs_guard) {
        needs_guard = false;
        first = n->init;
        if (depends_on(first, inner)) {
            needs_guard = true;
            first = invariant_part(first, o_max, n->iterator);
        }
        expr up = n->upper;
        if (depends_on(up, inner)) {
            needs_guard = true;
            up = invariant_part(up, o_min, n->iterator);
        }
        return lir::simplify(lir::simplify(up - first) + 1);
    }

    // ---- barriers of cache_shared.  Every LDS tile comes with a barrier before its cooperative copy (the
    // previous contents are no longer read) and one after it (the new contents are visible), in the
    // reference's order (tiramisu_core.cpp:9479-9515): two tiles filled at the same loop level give
    //   sync  copy(B)  sync  sync  copy(A)  sync  compute.
    // Copies of different tiles that read global memory only do not need a barrier between them, and two
    // barriers in a row are one: the sequence is emitted as  sync  copy(B)  copy(A)  sync  compute.
    static bool is_sync(const node_ptr &n) { return n->kind == node_kind::leaf && n->lkind == leaf_kind::sync; }

    // the LDS tiles written by a statement list that consists of cooperative cache copies only (else: false)
    bool tiles_filled_by(const std::vector<node_ptr> &nodes, std::set<std::string> &tiles) const {
        bool only_copies = !nodes.empty();
        for (auto &n : nodes)
            lir::walk(n, [&](const node_ptr &x) {
                if (x->kind != node_kind::leaf) return;
                if (x->lkind != leaf_kind::assign || !x->comp || !x->comp->get_cache_consumer() || !x->lhs ||
                    x->lhs->get_location() != memory_location::shared) { only_copies = false; return; }
                x->rhs.visit([&](const expr &e) {
                    if (e.get_expr_type() == e_op && e.get_op_type() == o_access &&
                        f->get_buffers().at(e.get_name())->get_location() == memory_location::shared) only_copies = false;
                });
                tiles.insert(x->lhs->get_name());
            });
        return only_copies;
    }

    std::vector<node_ptr> without_redundant_barriers(const std::vector<node_ptr> &in) const {
        if (backend_option("TIRAMISU_HIP_KEEP_BARRIERS")) return in;
        std::vector<node_ptr> flat, v;
        std::function<void(const node_ptr &)> flatten = [&](const node_ptr &n) {
            if (n && n->kind == node_kind::block) for (auto &c : n->children) flatten(c);
            else if (n) flat.push_back(n);
        };
        for (auto &n : in) flatten(n);
        for (auto &n : flat)
            if (!(is_sync(n) && !v.empty() && is_sync(v.back()))) v.push_back(n);      // two barriers in a row
        for (bool changed = true; changed;) {
            changed = false;
            std::vector<size_t> syncs;
            for (size_t i = 0; i < v.size(); i++) if (is_sync(v[i])) syncs.push_back(i);
            for (size_t s = 1; s + 1 < syncs.size() && !changed; s++) {
                std::set<std::string> before, after;
                const std::vector<node_ptr> left(v.begin() + syncs[s - 1] + 1, v.begin() + syncs[s]), right(v.begin() + syncs[s] + 1, v.begin() + syncs[s + 1]);
                if (!tiles_filled_by(left, before) || !tiles_filled_by(right, after)) continue;
                bool disjoint = true;
                for (auto &t : before) if (after.count(t)) disjoint = false;
                if (!disjoint) continue;
                v.erase(v.begin() + syncs[s]);
                changed = true;
            }
        }
        return v;
    }

    // ---- statements that no thread loop encloses.  The program means them to run once per iteration of the loops
    // around them (sequential semantics; on the CPU they do), but every thread of the workgroup reaches them: stores
    // of the same value are merely repeated, an accumulation (x = x + ...) is wrong -- the reference's CUDA printer
    // emits them as they stand (tiramisu_codegen_cuda.cpp: a thread loop becomes an index and a guard, what lies
    // outside it is code of every thread).  Here a statement or loop nest outside all thread loops that writes memory
    // the other threads see (global, LDS) runs on the workgroup's first thread, between two barriers: what the
    // thread loops before it wrote is there, and what it writes is there for the thread loops after it.  The barriers
    // are reached by all threads: nothing thread-dependent encloses such a statement.  Statements that write a
    // thread's own registers or arrays stay as they are -- every thread needs them.
    std::set<const node *> once_per_workgroup;       // roots of such subtrees (filled by mark_once_per_workgroup)
    bool kernel_has_thread_loops() const { return loops_per_dim[1][0] + loops_per_dim[1][1] + loops_per_dim[1][2] > 0; }
    bool may_run_on_one_thread(const node_ptr &n) const {
        bool ok = true, writes = false;
        lir::walk(n, [&](const node_ptr &x) {
            if (x->kind == node_kind::loop && (x->gpu_thread >= 0 || x->gpu_block >= 0)) ok = false;
            if (x->kind != node_kind::leaf) return;
            if (x->lkind == leaf_kind::call) { writes = true; return; }
            if (x->lkind != leaf_kind::assign || !x->lhs) { ok = false; return; }      // declarations, lets, barriers, copies
            const memory_location where = x->lhs->get_location();
            if (where == memory_location::global || where == memory_location::host || where == memory_location::shared) writes = true;
            else ok = false;
        });
        return ok && writes;
    }
    void mark_once_per_workgroup(const node_ptr &n) {
        if (!n || backend_option("TIRAMISU_HIP_EVERY_THREAD_RUNS_ALL")) return;
        if (n->kind == node_kind::loop && n->gpu_thread >= 0) return;               // below a thread loop everything is per thread
        if (n->kind != node_kind::block && may_run_on_one_thread(n)) { once_per_workgroup.insert(n.get()); return; }
        for (auto &c : n->children) mark_once_per_workgroup(c);
        mark_once_per_workgroup(n->body);
        mark_once_per_workgroup(n->then_body);
        mark_once_per_workgroup(n->else_body);
    }
    void emit_on_first_thread(const std::vector<node_ptr> &nodes, int ind) {
        std::string first;
        for (int d = 0; d < 3; d++)
            if (loops_per_dim[1][d] > 0) first += std::string(first.empty() ? "" : " && ") + "threadIdx." + "xyz"[d] + " == 0";
        body << pad(ind) << "__syncthreads();\n";
        body << pad(ind) << "if (" << first << ") {   // once per workgroup: no thread loop around these statements\n";
        for (auto &c : nodes) emit_node(c, ind + 1);
        body << pad(ind) << "}\n";
        body << pad(ind) << "__syncthreads();\n";
        statements_on_first_thread = true;
    }
    bool statements_on_first_thread = false;
    bool conflicting_tags = false;

    void emit(const node_ptr &n, int ind) {
        if (!n) return;
        if (n->kind == node_kind::block) {
            // neighbours that run once share one pair of barriers
            std::vector<node_ptr> run;
            for (auto &c : without_redundant_barriers(n->children)) {
                if (once_per_workgroup.count(c.get())) { run.push_back(c); continue; }
                if (!run.empty()) { emit_on_first_thread(run, ind); run.clear(); }
                emit(c, ind);
            }
            if (!run.empty()) emit_on_first_thread(run, ind);
            return;
        }
        if (once_per_workgroup.count(n.get())) { emit_on_first_thread({n}, ind); return; }
        emit_node(n, ind);
    }

    void emit_node(const node_ptr &n, int ind) {
        if (!n) return;
        switch (n->kind) {
        case node_kind::block:
            for (auto &c : without_redundant_barriers(n->children)) emit(c, ind);
            break;
        case node_kind::cond:
            body << pad(ind) << "if (" << dev.print(n->condition) << ") {\n";
            emit(n->then_body, ind + 1);
            if (n->else_body) {
                body << pad(ind) << "} else {\n";
                emit(n->else_body, ind + 1);
            }
            body << pad(ind) << "}\n";
            break;
        case node_kind::loop: emit_loop(n, ind); break;
        case node_kind::leaf: emit_leaf(n, ind); break;
        }
    }

    void emit_loop(const node_ptr &n, int ind) {
        const bool is_block = n->gpu_block >= 0, is_thread = n->gpu_thread >= 0;
        auto red = reductions.find(n.get());
        if (red != reductions.end()) {
            emit_thread_reduction(n, red->second, ind);
            return;
        }
        if (is_thread && (predicated_loops.count(n.get()) || (!live_predicates.empty() && holds_wide_reduction(n)))) {
            const int dim = n->gpu_thread;
            bool guard;
            expr first;
            block_ext[dim].push_back(host_extent(n, first, guard));
            if (loops_per_dim[1][dim] > 1 || predicated_loops.count(n.get())) guard = true;
            body << pad(ind) << "{\n";
            body << pad(ind + 1) << "const int32_t " << n->iterator << " = (int32_t)threadIdx." << "xyz"[dim] << " + " << dev.print(first) << ";\n";
            if (guard) {
                body << pad(ind + 1) << "const bool _live_" << n->iterator << " = " << n->iterator << " >= " << dev.print(n->init) << " && " << n->iterator
                     << " <= " << dev.print(n->upper) << ";   // a predicate, not a branch: the sum below has a barrier that every thread must reach\n";
                live_predicates.push_back("_live_" + n->iterator);
            }
            emit_predicated(n->body, ind + 1);
            if (guard) live_predicates.pop_back();
            body << pad(ind) << "}\n";
            return;
        }
        if (retile.on && (is_block || is_thread)) {
            const int dim = is_block ? n->gpu_block : n->gpu_thread;
            bool guard;
            expr first;
            const expr ext = host_extent(n, first, guard);
            const long S = retile.tile[dim], wide = retile.wide[dim];
            body << pad(ind) << "{\n";
            if (is_block) {
                grid_ext[dim].push_back(lir::simplify((ext * expr((int32_t)S) + expr((int32_t)(wide - 1))) / expr((int32_t)wide)));
                body << pad(ind + 1) << "const uint32_t _g" << dim << " = " << (fast_block_dim >= 0 ? "_tile." : "blockIdx.") << "xyz"[dim] << " * " << wide
                     << "u + threadIdx." << "xyz"[dim] << ";   // the point's index along this dimension\n";
                body << pad(ind + 1) << "const int32_t " << n->iterator << " = (int32_t)(_g" << dim << " / " << S << "u);\n";
                body << pad(ind + 1) << "if (" << n->iterator << " <= " << dev.print(n->upper) << ") {\n";
                guard = true;
            } else {
                block_ext[dim].push_back(expr((int32_t)wide));
                body << pad(ind + 1) << "const int32_t " << n->iterator << " = (int32_t)(_g" << dim << " % " << S << "u);\n";
                if (guard)
                    body << pad(ind + 1) << "if (" << n->iterator << " >= " << dev.print(n->init) << " && " << n->iterator
                         << " <= " << dev.print(n->upper) << ") {\n";
            }
            emit(n->body, ind + (guard ? 2 : 1));
            if (guard) body << pad(ind + 1) << "}\n";
            body << pad(ind) << "}\n";
            return;
        }
        if (is_block || is_thread) {
            const int dim = is_block ? n->gpu_block : n->gpu_thread;
            bool guard;
            expr first;
            expr ext = host_extent(n, first, guard);
            (is_block ? grid_ext : block_ext)[dim].push_back(ext);
            if (loops_per_dim[is_block ? 0 : 1][dim] > 1) guard = true;
            const char *idx = is_block ? (fast_block_dim >= 0 ? "_tile." : "blockIdx.") : "threadIdx.";
            body << pad(ind) << "{\n";
            body << pad(ind + 1) << "const int32_t " << n->iterator << " = (int32_t)" << idx << "xyz"[dim] << " + "
                 << dev.print(first) << ";\n";
            if (guard)
                body << pad(ind + 1) << "if (" << n->iterator << " >= " << dev.print(n->init) << " && " << n->iterator
                     << " <= " << dev.print(n->upper) << ") {\n";
            emit(n->body, ind + (guard ? 2 : 1));
            if (guard) body << pad(ind + 1) << "}\n";
            body << pad(ind) << "}\n";
            return;
        }
        // Short loops are unrolled (register tiles are arrays that must end up in registers, and index arithmetic folds),
        // but within a budget: the statements that unrolling this loop and every short loop below it would lay out.
        // Beyond it the loop is left to the compiler's own judgement -- nests of many short loops (tensor contractions
        // over spin and colour indices: 3 x 2 x 3 x 2 x 8 x 3 x 2) would otherwise become tens of thousands of
        // statements, minutes of device compilation and code that misses the instruction cache.
        expr lo = lir::simplify(n->init), up = lir::simplify(n->upper);
        const bool small_loop = lo.is_integer_literal() && up.is_integer_literal() && up.get_int_val() - lo.get_int_val() < 32;
        const bool small = small_loop && unrolled_statements(n) <= unroll_budget();
        if (n->unrolled || small) body << pad(ind) << "#pragma unroll\n";
        body << pad(ind) << "for (int32_t " << n->iterator << " = " << dev.print(n->init) << "; " << n->iterator
             << " <= " << dev.print(n->upper) << "; " << n->iterator << " += " << dev.print(n->increment) << ") {\n";
        emit(n->body, ind + 1);
        body << pad(ind) << "}\n";
    }

    long unroll_budget() const {
        const char *e = backend_option("TIRAMISU_HIP_UNROLL_BUDGET");
        return e ? std::atol(e) : 1024;
    }
    // statements of the loop nest below n with every loop of constant extent unrolled (other loops count once)
    static long unrolled_statements(const node_ptr &n) {
        if (!n) return 0;
        switch (n->kind) {
        case node_kind::leaf: return n->lkind == leaf_kind::assign || n->lkind == leaf_kind::call ? 1 : 0;
        case node_kind::block: { long s = 0; for (auto &c : n->children) s += unrolled_statements(c); return s; }
        case node_kind::cond: return unrolled_statements(n->then_body) + unrolled_statements(n->else_body);
        case node_kind::loop: {
            const expr lo = lir::simplify(n->init), up = lir::simplify(n->upper);
            long trip = 1;
            if (n->gpu_block < 0 && n->gpu_thread < 0 && lo.is_integer_literal() && up.is_integer_literal())
                trip = std::max<long>(1, up.get_int_val() - lo.get_int_val() + 1);
            const long below = unrolled_statements(n->body);
            return below > (1L << 40) / trip ? (1L << 40) : trip * below;
        }
        }
        return 0;
    }

    long shared_bytes = 0;      // of the __shared__ arrays declared so far in this kernel
    std::string declaration(const buffer *b) {
        std::string t = primitive_c_name(b->get_elements_type());
        switch (b->get_location()) {
        case memory_location::reg: return t + " " + b->get_name() + ";";
        case memory_location::local:
        case memory_location::shared: {
            if (!b->has_constant_extents())
                ERROR("buffer " + b->get_name() + " lives in a GPU kernel and needs constant extents", true);
            long cnt = 1;
            for (auto &d : b->get_dim_sizes()) cnt *= lir::simplify(d).get_int_val();
            if (b->get_location() == memory_location::shared) shared_bytes += cnt * (long)primitive_size(b->get_elements_type());
            return std::string(b->get_location() == memory_location::shared ? "__shared__ " : "") + t + " " +
                   b->get_name() + "[" + std::to_string(cnt) + "];";
        }
        default:
            ERROR("buffer " + b->get_name() + " is allocated inside a GPU kernel but is neither shared, local nor register", true);
        }
        return "";
    }

    void emit_leaf(const node_ptr &n, int ind) {
        if (n.get() == pending_leaf) {
            body << pad(ind) << pending_partial << " = " << pending_combine(pending_partial, dev.print(pending_term)) << ";\n";
            return;
        }
        switch (n->lkind) {
        case leaf_kind::sync: body << pad(ind) << "__syncthreads();\n"; return;
        case leaf_kind::allocate:
            declared.insert(n->target->get_name());
            body << pad(ind) << declaration(n->target) << "\n";
            return;
        case leaf_kind::release: return;
        case leaf_kind::copy: ERROR("memcpy computation " + n->comp->get_name() + " is scheduled inside a GPU kernel", true);
        case leaf_kind::let:
            // visible to the statements that follow in this loop body
            body << pad(ind) << "const " << primitive_c_name(n->comp->get_data_type()) << " " << n->comp->get_name() << " = "
                 << dev.print(n->rhs) << ";\n";
            return;
        default: break;
        }
        int i2 = ind;
        const bool scoped = !n->lets.empty() || n->predicate.is_defined();
        if (scoped) { body << pad(ind) << "{\n"; i2++; }
        for (auto &l : n->lets)
            body << pad(i2) << "const " << primitive_c_name(l.second.get_data_type()) << " " << l.first << " = "
                 << dev.print(l.second) << ";\n";
        if (n->predicate.is_defined()) { body << pad(i2) << "if (" << dev.print(n->predicate) << ") {\n"; i2++; }
        if (n->lhs) body << pad(i2) << dev.store(n->lhs, n->lhs_index, dev.print(n->rhs), n->rhs.get_data_type()) << "\n";
        else body << pad(i2) << dev.print(n->rhs) << ";\n";
        if (n->predicate.is_defined()) { i2--; body << pad(i2) << "}\n"; }
        if (scoped) body << pad(ind) << "}\n";
    }
};

std::string max_text(const std::vector<expr> &v, const c_printer &host) {
    if (v.empty()) return "1";
    bool all_lit = true;
    long m = 0;
    for (auto &e : v) {
        if (e.is_integer_literal()) m = std::max<long>(m, e.get_int_val());
        else all_lit = false;
    }
    if (all_lit) return std::to_string(m);
    std::string s = host.print(v[0]);
    for (size_t i = 1; i < v.size(); i++) s = "t_max(" + s + ", " + host.print(v[i]) + ")";
    return "(uint32_t)t_max((int32_t)0, (int32_t)(" + s + "))";
}

}  // namespace

static kernel emit_generic_kernel_impl(context &ctx, const node_ptr &root, const fusion_request *batch, bool &batch_ok);

kernel emit_generic_kernel(context &ctx, const node_ptr &root) {
    bool ok = true;
    return emit_generic_kernel_impl(ctx, root, nullptr, ok);
}

kernel emit_generic_kernel_batched(context &ctx, const node_ptr &root, const fusion_request &batch, bool &ok) {
    const int first_id = context::peek_next_kernel_id();
    ok = true;
    kernel k = emit_generic_kernel_impl(ctx, root, &batch, ok);
    if (!ok) context::set_next_kernel_id(first_id);
    return k;
}

static kernel emit_generic_kernel_impl(context &ctx, const node_ptr &root, const fusion_request *batch, bool &batch_ok) {
    generic_kernel_gen g(ctx);
    g.prepass(root);
    g.emit(root, 1);

    kernel k;
    k.how = "generic";
    if (g.lanes_renumbered) k.how += ", threadIdx.x given to the thread loop along which the accesses have unit stride";
    if (g.retile.on)
        k.how += ", points dealt out again to workgroups of " + std::to_string(g.retile.wide[0]) + " x " + std::to_string(g.retile.wide[1]) +
                 " (the program's tiles: " + std::to_string(g.retile.tile[0]) + " x " + std::to_string(g.retile.tile[1]) + ")";
    if (g.fast_block_dim >= 0) k.how += std::string(", workgroups renumbered: an eighth of the tiles per XCD, ") + "xy"[g.fast_block_dim] + " fastest";
    if (g.wave_reductions)
        k.how += ", " + std::to_string(g.wave_reductions) + " sum(s) across the threads of a loop lowered to DPP wavefront reductions" +
                 (g.needs_reduction_scratch ? " (wavefront totals combined through LDS)" : "");
    if (g.conflicting_tags) k.how += ", a loop tagged as a block dimension by some statements and as a thread dimension by others is a block dimension";
    if (g.statements_on_first_thread) k.how += ", statements outside the thread loops run on the workgroup's first thread between barriers";
    k.name = "_kernel_" + std::to_string(ctx.next_kernel_id());
    function *f = ctx.f;

    // parameters: free scalars sorted by name, then global buffers sorted by name
    // (reference: tiramisu_codegen_cuda.cpp:1324-1331)
    c_printer host;
    host.fct = f;
    std::set<std::string> extent_scalars, extent_buffers;
    host.used_scalars = &extent_scalars;
    host.used_buffers = &extent_buffers;
    for (int d = 0; d < 3; d++) {
        k.grid[d] = max_text(g.grid_ext[d], host);
        k.block[d] = max_text(g.block_ext[d], host);
    }
    std::vector<std::string> top_decls;
    bool batch_iterator_used = false;
    if (batch) {
        // the nest's own grid must leave z free and must not depend on the iteration
        if (k.grid[2] != "1" || extent_scalars.count(batch->batch_iterator)) { batch_ok = false; return k; }
        k.how += ", iterations of the parallel host loop as gridDim.z";
        c_printer hp;
        hp.fct = f;
        k.batch_first = hp.print(batch->batch_first);
        k.grid[2] = "((" + hp.print(batch->batch_last) + ") >= _batch_first ? (" + hp.print(batch->batch_last) + ") - _batch_first + 1 : 0)";
        k.params.push_back({false, "_batch_first", p_int32});            // as the launch declares it
    }
    for (auto &nm : g.used_scalars) {
        if (g.inner.count(nm)) continue;
        if (batch && nm == batch->batch_iterator) { batch_iterator_used = true; continue; }
        // An iterator of a host loop around the launch: host loops are declared int32_t whatever the program's loop
        // iterator type is (set_loop_iterator_type(p_int64) types the expressions, not the generated loops), and the
        // launch passes the variable's address -- the parameter must have the variable's own width.
        primitive_t t = p_int32;
        for (auto c : f->get_invariants())
            if (c->get_name() == nm) t = c->get_data_type();
        for (auto c : f->get_computation_by_name(nm))   // a constant scheduled on the host
            if (c->is_let_stmt()) t = c->get_data_type();
        k.params.push_back({false, nm, t});
    }
    for (auto &nm : g.used_buffers) {
        buffer *b = f->get_buffers().at(nm);
        switch (b->get_location()) {
        case memory_location::global: k.params.push_back({true, nm, b->get_elements_type()}); break;
        case memory_location::host: {
            if (!f->copies_host_buffers_implicitly())
                ERROR("buffer " + nm + " is used inside a GPU kernel but lives in host memory; tag it with tag_gpu_global() "
                      "and copy it with memcpy()", true);
            bool written = false;
            lir::walk(root, [&](const node_ptr &x) {
                if (x->kind == node_kind::leaf && x->lhs == b) written = true;
            });
            k.params.push_back({true, nm, b->get_elements_type()});
            k.host_mirrors.push_back({nm, primitive_c_name(b->get_elements_type()),
                                      "(uint64_t)(" + host.element_count(b) + ") * sizeof(" + primitive_c_name(b->get_elements_type()) + ")", written});
            break;
        }
        case memory_location::constant:
            // a file-scope __constant__ array of the code object: not a parameter
            // (reference: tiramisu_codegen_cuda.cpp:811-829, :1192-1193)
            ctx.constant_buffers.insert(nm);
            break;
        default:
            if (!g.declared.count(nm)) top_decls.push_back(g.declaration(b));
        }
    }

    std::ostringstream os;
    long threads = 1;
    bool lit = true;
    for (int d = 0; d < 3; d++) {
        char *end = nullptr;
        long v = strtol(k.block[d].c_str(), &end, 10);
        if (end && *end == 0) threads *= v; else lit = false;
    }
    // What the hardware will refuse at the launch is refused here, where the program can still be named (the device
    // compiler accepts both): more than 1024 threads in a workgroup, more than 160 KiB of LDS.
    if (lit && threads > 1024)
        ERROR("kernel " + k.name + " of " + f->get_name() + ": a workgroup of " + k.block[0] + " x " + k.block[1] + " x " + k.block[2] + " = " +
              std::to_string(threads) + " threads; the limit is 1024", true);
    const long lds = g.shared_bytes + (g.needs_reduction_scratch ? (g.wide_reduction_scratch ? 128 : 64) : 0);
    if (lds > 160 * 1024)
        ERROR("kernel " + k.name + " of " + f->get_name() + ": " + std::to_string(lds) + " bytes of shared memory; a workgroup has 163840", true);
    os << "extern \"C\" __global__ void ";
    if (lit) os << "__launch_bounds__(" << threads << ") ";
    os << k.name << "(";
    for (size_t i = 0; i < k.params.size(); i++) {
        auto &p = k.params[i];
        os << (i ? ", " : "");
        if (p.is_buffer) os << primitive_c_name(p.type) << " *__restrict__ " << p.name;
        else os << "const " << primitive_c_name(p.type) << " " << p.name;
    }
    os << ")\n{\n";
    if (batch && batch_iterator_used)
        os << "    const " << primitive_c_name(global::get_loop_iterator_data_type()) << " " << batch->batch_iterator << " = (int32_t)blockIdx.z + _batch_first;\n";
    for (auto &d : top_decls) os << "    " << d << "\n";
    if (g.needs_reduction_scratch) os << "    __shared__ " << (g.wide_reduction_scratch ? "double" : "float") << " _reduction_scratch[16];\n";
    if (g.fast_block_dim >= 0) {
        // hardware order l (x fastest) -> XCD l % XCDS, its (l / XCDS)-th workgroup -> tile t of the XCD's share
        const char fast = "xy"[g.fast_block_dim], slow = "xy"[1 - g.fast_block_dim];
        os << "    uint3 _tile;\n    {\n"
           << "        const unsigned _n = gridDim.x * gridDim.y, _l = blockIdx.x + gridDim.x * blockIdx.y;\n"
           << "        const unsigned _c = _l % " << ttarget::XCDS << "u, _share = _n / " << ttarget::XCDS << "u, _extra = _n % " << ttarget::XCDS << "u;\n"
           << "        const unsigned _t = _c * _share + (_c < _extra ? _c : _extra) + _l / " << ttarget::XCDS << "u;\n";
        os << "        _tile." << fast << " = _t % gridDim." << fast << ";\n        _tile." << slow << " = _t / gridDim." << fast << ";\n"
           << "        _tile.z = 0;\n    }\n";
    }
    os << g.body.str() << "}\n";
    k.source = os.str();
    return k;
}

std::string launch_text(const kernel &k, const std::string &ind_outer) {
    std::ostringstream os;
    std::string ind = ind_outer;
    if (!k.host_mirrors.empty()) {
        // implicit copies: inside the inner scope the buffer's name means its device copy
        os << ind << "{\n";
        for (auto &m : k.host_mirrors) os << ind << "    " << m.ctype << " *" << m.name << "__host = " << m.name << ";\n";
        os << ind << "    {\n";
        ind += "        ";
        for (auto &m : k.host_mirrors) {
            os << ind << m.ctype << " *" << m.name << " = (" << m.ctype << " *)tiramisu_hip_malloc(" << m.bytes << ");\n";
            os << ind << "tiramisu_hip_memcpy_to_device((void *)" << m.name << ", (void *)" << m.name << "__host, " << m.bytes << ");\n";
        }
    }
    os << ind << "{\n";
    if (!k.batch_first.empty()) os << ind << "    const int32_t _batch_first = " << k.batch_first << ";\n";
    os << ind << "    void *_args[] = {";
    for (size_t i = 0; i < k.params.size(); i++) os << (i ? ", " : "") << "(void *)&" << k.params[i].name;
    if (k.params.empty()) os << "nullptr";
    os << "};\n";
    os << ind << "    const uint32_t _grid[3] = {(uint32_t)(" << k.grid[0] << "), (uint32_t)(" << k.grid[1] << "), (uint32_t)("
       << k.grid[2] << ")};\n";
    os << ind << "    const uint32_t _block[3] = {(uint32_t)(" << k.block[0] << "), (uint32_t)(" << k.block[1]
       << "), (uint32_t)(" << k.block[2] << ")};\n";
    os << ind << "    static void *_fn = tiramisu_hip_module_get_function(_tiramisu_module(), \"" << k.name << "\");\n";
    os << ind << "    tiramisu_hip_launch(_fn, _grid, _block, (uint32_t)(" << k.lds_bytes << "), _args);\n";
    os << ind << "}\n";
    if (!k.host_mirrors.empty()) {
        for (auto &m : k.host_mirrors) {
            if (m.written)
                os << ind << "tiramisu_hip_memcpy_to_host((void *)" << m.name << "__host, (void *)" << m.name << ", " << m.bytes << ");\n";
            os << ind << "tiramisu_hip_free((void *)" << m.name << ");\n";
        }
        os << ind_outer << "    }\n" << ind_outer << "}\n";
    }
    return os.str();
}

namespace {

// ---------------------------------------------------------------- host glue

struct host_gen {
    context &ctx;
    function *f;
    c_printer hp;
    std::ostringstream out;
    std::set<std::string> extern_calls;
    std::vector<std::string> extern_decls;
    std::vector<node *> loop_stack;

    host_gen(context &c) : ctx(c), f(c.f) { hp.fct = f; }

    // A host loop tagged parallel is handed to the runtime's pool when its iterations can run
    // side by side as emitted: unit stride, not nested in another such loop, and no buffer
    // allocated or released in its body (those assign variables of the enclosing function).
    bool in_parallel_loop = false;
    int parallel_loops = 0;
    bool runs_in_parallel(const node_ptr &n) const {
        if (!n->parallel || in_parallel_loop || backend_option("TIRAMISU_HIP_SERIAL_HOST_LOOPS")) return false;
        const expr inc = lir::simplify(n->increment);
        if (!inc.is_integer_literal() || inc.get_int_val() != 1) return false;
        bool ok = true;
        lir::walk(n->body, [&](const node_ptr &x) {
            if (x->kind == node_kind::leaf && (x->lkind == leaf_kind::allocate || x->lkind == leaf_kind::release)) ok = false;
        });
        return ok;
    }

    static bool is_gpu_loop(const node_ptr &n) { return n->kind == node_kind::loop && (n->gpu_block >= 0 || n->gpu_thread >= 0); }

    void require_host(const buffer *b, const std::string &who) {
        if (b->get_location() != memory_location::host)
            ERROR("computation " + who + " runs on the host but touches GPU buffer " + b->get_name() +
                  "; map its loops to the GPU (gpu_tile / tag_gpu_level)", true);
    }

    void declare_call(const expr &call) {
        const std::string &nm = call.get_name();
        if (nm.rfind("tiramisu_hip_", 0) == 0 || extern_calls.count(nm)) return;
        extern_calls.insert(nm);
        std::string s = "extern \"C\" " + primitive_c_name(call.get_data_type()) + " " + nm + "(";
        for (size_t i = 0; i < call.get_arguments().size(); i++) {
            const expr &a = call.get_arguments()[i];
            std::string t = (a.get_expr_type() == e_op && a.get_op_type() == o_buffer) ? "void *"
                            : (a.get_expr_type() == e_op && a.get_op_type() == o_address) ? "halide_buffer_t *"
                            : primitive_c_name(a.get_data_type());
            s += (i ? ", " : "") + t;
        }
        extern_decls.push_back(s + ");");
    }

    void emit(const node_ptr &n, int ind) {
        if (!n) return;
        switch (n->kind) {
        case node_kind::block:
            emit_sequence(n->children, ind);
            break;
        case node_kind::cond:
            out << pad(ind) << "if (" << hp.print(n->condition) << ") {\n";
            emit(n->then_body, ind + 1);
            if (n->else_body) {
                out << pad(ind) << "} else {\n";
                emit(n->else_body, ind + 1);
            }
            out << pad(ind) << "}\n";
            break;
        case node_kind::loop:
            if (is_gpu_loop(n)) {
                emit_kernel_nest(n, ind);
            } else {
                // a time loop around a stencil nest may be taken over as a whole
                launch_plan plan;
                if (emit_stencil(ctx, nullptr, n, plan)) {
                    for (auto &k : plan.kernels) ctx.kernels.push_back(k);
                    out << plan.host_code;
                    break;
                }
                if (runs_in_parallel(n) && emit_batched(n, ind)) break;
                if (runs_in_parallel(n) && emit_distributed(n, ind)) break;
                if (runs_in_parallel(n)) {
                    // iterations on pool threads, each with a stream of its own (what the reference's
                    // Halide parallel loop around kernel calls does: tiramisu_codegen_halide.cpp:2104-2145)
                    const std::string body = "_parallel_body_" + std::to_string(parallel_loops++);
                    out << pad(ind) << "{\n";
                    out << pad(ind + 1) << "auto " << body << " = [&](int32_t " << n->iterator << ") {\n";
                    in_parallel_loop = true;
                    ctx.host_iterators.push_back(n->iterator);
                    emit(n->body, ind + 2);
                    ctx.host_iterators.pop_back();
                    in_parallel_loop = false;
                    out << pad(ind + 1) << "};\n";
                    out << pad(ind + 1) << "tiramisu_hip_parallel_for(" << hp.print(n->init) << ", " << hp.print(n->upper)
                        << ", [](int32_t _i, void *_p) { (*static_cast<decltype(" << body << ") *>(_p))(_i); }, (void *)&" << body << ");\n";
                    out << pad(ind) << "}\n";
                    break;
                }
                out << pad(ind) << "for (int32_t " << n->iterator << " = " << hp.print(n->init) << "; " << n->iterator
                    << " <= " << hp.print(n->upper) << "; " << n->iterator << " += " << hp.print(n->increment) << ") {\n";
                ctx.host_iterators.push_back(n->iterator);
                emit(n->body, ind + 1);
                ctx.host_iterators.pop_back();
                out << pad(ind) << "}\n";
            }
            break;
        case node_kind::leaf: emit_leaf(n, ind); break;
        }
    }

    void take(launch_plan &plan, int ind) {
        for (auto &k : plan.kernels) ctx.kernels.push_back(k);
        if (!plan.host_code.empty()) out << plan.host_code;
        else for (auto &k : plan.kernels) out << launch_text(k, pad(ind));
    }

    // Statements in order.  A contraction nest directly followed by another GPU-mapped nest is offered
    // to the contraction emitter as a pair: a point-wise consumer of the result runs in the same kernel.
    void emit_sequence(const std::vector<node_ptr> &nodes, int ind) {
        for (size_t i = 0; i < nodes.size(); i++) {
            if (i + 1 < nodes.size() && is_gpu_loop(nodes[i]) && is_gpu_loop(nodes[i + 1])) {
                fusion_request req;
                req.consumer = nodes[i + 1];
                launch_plan plan;
                const int first_id = context::peek_next_kernel_id();
                if (emit_contraction(ctx, nodes[i], plan, &req)) {
                    take(plan, ind);
                    i++;
                    continue;
                }
                context::set_next_kernel_id(first_id);
            }
            emit(nodes[i], ind);
        }
    }

    // A host loop tagged parallel whose body is nothing but GPU-mapped nests that the contraction
    // emitter takes: its iterations become gridDim.z of one launch per kernel instead of launches of
    // their own on pool threads.  (Independence of the iterations is what the tag asserts; kernels of
    // the body still run one after the other, each over all iterations, which keeps every dependence
    // that the serial loop body had within an iteration.)
    bool emit_batched(const node_ptr &n, int ind) {
        if (backend_option("TIRAMISU_HIP_NO_BATCHED_LAUNCH")) return false;
        std::vector<node_ptr> nests;
        if (n->body && n->body->kind == node_kind::block) nests = n->body->children;
        else if (n->body) nests.push_back(n->body);
        if (nests.empty()) return false;
        for (auto &x : nests)
            if (!is_gpu_loop(x)) return false;
        const int first_id = context::peek_next_kernel_id();
        std::vector<launch_plan> plans;
        ctx.host_iterators.push_back(n->iterator);
        bool ok = true;
        for (size_t i = 0; i < nests.size() && ok; i++) {
            fusion_request req;
            req.batch_iterator = n->iterator;
            req.batch_first = n->init;
            req.batch_last = n->upper;
            launch_plan plan;
            if (i + 1 < nests.size()) {
                req.consumer = nests[i + 1];
                if (emit_contraction(ctx, nests[i], plan, &req)) { plans.push_back(plan); i++; continue; }
                req.consumer = nullptr;
                plan = launch_plan();
            }
            if (emit_contraction(ctx, nests[i], plan, &req)) plans.push_back(plan);
            else ok = false;
        }
        ctx.host_iterators.pop_back();
        if (!ok) {
            context::set_next_kernel_id(first_id);
            return false;
        }
        for (auto &p : plans) take(p, ind);
        return true;
    }

    // A host loop tagged parallel whose body is a sequence of library GEMM calls, kernels and serial loops around
    // them (the reference's library LSTM: per layer one batched input product, then per time step a recurrent
    // product and a point-wise kernel) is distributed over its statements: every statement runs for all
    // iterations of the parallel loop at once -- a kernel as one launch with the iterations as gridDim.z, GEMM
    // calls of one statement as one batched launch (tiramisu_hip_batch_begin / _end) -- in the order of the body,
    // on the calling thread's stream.  The tag asserts that iterations are independent, and the order of the
    // statements within an iteration is kept, so every dependence of the serial program holds; what it buys is
    // launches that fill the chip instead of one small launch per iteration on streams that slow each other
    // down.  Serial loops inside the body must not have bounds that involve the parallel iterator.
    bool distributable(const node_ptr &x, const std::string &it, int &gpu_statements) const {
        if (!x) return true;
        switch (x->kind) {
        case node_kind::block:
            for (auto &c : x->children)
                if (!distributable(c, it, gpu_statements)) return false;
            return true;
        case node_kind::cond: return false;
        case node_kind::loop: {
            if (is_gpu_loop(x)) {
                bool z_used = false;
                lir::walk(x, [&](const node_ptr &y) { if (y->kind == node_kind::loop && y->gpu_block == 2) z_used = true; });
                gpu_statements++;
                return !z_used;
            }
            if (x->parallel) return false;
            for (const expr &e : {x->init, x->upper, x->increment})
                if (e.is_defined() && lir::mentions(e, it)) return false;
            return distributable(x->body, it, gpu_statements);
        }
        case node_kind::leaf:
            if (x->lkind == leaf_kind::allocate || x->lkind == leaf_kind::release || x->lkind == leaf_kind::let || x->lkind == leaf_kind::copy) return false;
            if (is_library_gemm(x)) gpu_statements++;
            return true;
        }
        return false;
    }
    static bool is_library_gemm(const node_ptr &x) {
        bool gemm = false;
        if (x->kind == node_kind::leaf && x->rhs.is_defined())
            x->rhs.visit([&](const expr &e) {
                if (e.get_expr_type() == e_op && e.get_op_type() == o_call && (e.get_name() == "tiramisu_hip_sgemm" || e.get_name() == "tiramisu_hip_dgemm")) gemm = true;
            });
        return gemm;
    }
    void emit_for_all_iterations(const node_ptr &x, const node_ptr &par, int ind) {
        switch (x->kind) {
        case node_kind::block:
            for (auto &c : x->children) emit_for_all_iterations(c, par, ind);
            return;
        case node_kind::loop:
            if (is_gpu_loop(x)) {
                fusion_request req;
                req.batch_iterator = par->iterator;
                req.batch_first = par->init;
                req.batch_last = par->upper;
                ctx.host_iterators.push_back(par->iterator);
                launch_plan plan;
                if (emit_contraction(ctx, x, plan, &req)) {
                    take(plan, ind);
                } else {
                    bool ok = true;
                    kernel k = emit_generic_kernel_batched(ctx, x, req, ok);
                    if (!ok) ERROR("a kernel inside a distributed parallel host loop could not take the loop's iterations as gridDim.z", true);
                    ctx.kernels.push_back(k);
                    out << launch_text(k, pad(ind));
                }
                ctx.host_iterators.pop_back();
                return;
            }
            out << pad(ind) << "for (int32_t " << x->iterator << " = " << hp.print(x->init) << "; " << x->iterator
                << " <= " << hp.print(x->upper) << "; " << x->iterator << " += " << hp.print(x->increment) << ") {\n";
            ctx.host_iterators.push_back(x->iterator);
            emit_for_all_iterations(x->body, par, ind + 1);
            ctx.host_iterators.pop_back();
            out << pad(ind) << "}\n";
            return;
        case node_kind::leaf: {
            const bool gemm = is_library_gemm(x);
            if (gemm) out << pad(ind) << "tiramisu_hip_batch_begin();\n";
            out << pad(ind) << "for (int32_t " << par->iterator << " = " << hp.print(par->init) << "; " << par->iterator
                << " <= " << hp.print(par->upper) << "; " << par->iterator << " += 1) {\n";
            emit_leaf(x, ind + 1);
            out << pad(ind) << "}\n";
            if (gemm) out << pad(ind) << "tiramisu_hip_batch_end();\n";
            return;
        }
        default: return;
        }
    }
    bool emit_distributed(const node_ptr &n, int ind) {
        if (backend_option("TIRAMISU_HIP_NO_DISTRIBUTED_HOST_LOOPS")) return false;
        int gpu_statements = 0;
        if (!n->body || !distributable(n->body, n->iterator, gpu_statements) || gpu_statements == 0) return false;
        out << pad(ind) << "{   // parallel host loop " << n->iterator << ", distributed over its statements\n";
        emit_for_all_iterations(n->body, n, ind + 1);
        out << pad(ind) << "}\n";
        return true;
    }

    void emit_kernel_nest(const node_ptr &n, int ind) {
        launch_plan plan;
        if (emit_contraction(ctx, n, plan) || emit_stencil(ctx, n, nullptr, plan)) {
            take(plan, ind);
            return;
        }
        kernel k = emit_generic_kernel(ctx, n);
        ctx.kernels.push_back(k);
        out << launch_text(k, pad(ind));
    }

    void emit_leaf(const node_ptr &n, int ind) {
        switch (n->lkind) {
        case leaf_kind::sync: return;
        case leaf_kind::copy: {
            buffer *s = n->copy_from, *d = n->copy_to;
            auto on_device = [](const buffer *b) {
                return b->get_location() == memory_location::global || b->get_location() == memory_location::constant;
            };
            for (const buffer *b : {s, d})
                if (b->get_location() != memory_location::host && !on_device(b))
                    ERROR("memcpy computation " + n->comp->get_name() + ": buffer " + b->get_name() + " lives inside a kernel", true);
            bool sg = on_device(s), dg = on_device(d);
            std::string bytes = "(uint64_t)(" + hp.element_count(s) + ") * sizeof(" + primitive_c_name(s->get_elements_type()) + ")";
            const char *fn = (!sg && d->get_location() == memory_location::constant) ? "tiramisu_hip_memcpy_to_symbol"
                             : (!sg && dg) ? "tiramisu_hip_memcpy_to_device" : (sg && !dg) ? "tiramisu_hip_memcpy_to_host"
                             : (sg && dg) ? "tiramisu_hip_memcpy_device_to_device" : nullptr;
            if (fn) out << pad(ind) << fn << "((void *)" << d->get_name() << ", (void *)" << s->get_name() << ", " << bytes << ");\n";
            else out << pad(ind) << "memcpy((void *)" << d->get_name() << ", (void *)" << s->get_name() << ", " << bytes << ");\n";
            return;
        }
        case leaf_kind::allocate: {
            buffer *b = n->target;
            std::string t = primitive_c_name(b->get_elements_type());
            std::string bytes = "(uint64_t)(" + hp.element_count(b, n->iterators) + ") * sizeof(" + t + ")";
            if (b->get_location() == memory_location::global)
                out << pad(ind) << b->get_name() << " = (" << t << " *)tiramisu_hip_malloc(" << bytes << ");\n";
            else if (b->get_location() == memory_location::host)
                out << pad(ind) << b->get_name() << " = (" << t << " *)malloc(" << bytes << ");\n";
            else
                ERROR("allocation of " + b->get_name() + " (a shared/local/register buffer) is scheduled outside a GPU kernel", true);
            return;
        }
        case leaf_kind::release: {
            buffer *b = n->target;
            if (b->get_location() == memory_location::global) out << pad(ind) << "tiramisu_hip_free((void *)" << b->get_name() << ");\n";
            else out << pad(ind) << "free((void *)" << b->get_name() << ");\n";
            return;
        }
        default: break;
        }
        if (n->lkind == leaf_kind::let) {
            out << pad(ind) << "const " << primitive_c_name(n->comp->get_data_type()) << " " << n->comp->get_name() << " = "
                << hp.print(n->rhs) << ";\n";
            return;
        }
        // host-side assignment or call
        n->rhs.visit([&](const expr &e) {
            if (e.get_expr_type() == e_op && e.get_op_type() == o_access) require_host(f->get_buffers().at(e.get_name()), n->comp->get_name());
            if (e.get_expr_type() == e_op && e.get_op_type() == o_call) declare_call(e);
        });
        if (n->lhs) require_host(n->lhs, n->comp->get_name());
        int i2 = ind;
        const bool scoped = !n->lets.empty() || n->predicate.is_defined();
        if (scoped) { out << pad(ind) << "{\n"; i2++; }
        for (auto &l : n->lets)
            out << pad(i2) << "const " << primitive_c_name(l.second.get_data_type()) << " " << l.first << " = " << hp.print(l.second) << ";\n";
        if (n->predicate.is_defined()) { out << pad(i2) << "if (" << hp.print(n->predicate) << ") {\n"; i2++; }
        if (n->lhs) out << pad(i2) << hp.store(n->lhs, n->lhs_index, hp.print(n->rhs), n->rhs.get_data_type()) << "\n";
        else out << pad(i2) << hp.print(n->rhs) << ";\n";
        if (n->predicate.is_defined()) { i2--; out << pad(i2) << "}\n"; }
        if (scoped) out << pad(ind) << "}\n";
    }
};

void collect_used_buffers(const node_ptr &root, std::set<std::string> &used) {
    lir::walk(root, [&](const node_ptr &n) {
        auto scan = [&](const expr &e) {
            if (!e.is_defined()) return;
            e.visit([&](const expr &x) {
                if (x.get_expr_type() == e_op && (x.get_op_type() == o_access || x.get_op_type() == o_buffer || x.get_op_type() == o_address_of))
                    used.insert(x.get_name());
            });
        };
        if (n->kind != node_kind::leaf) return;
        if (n->lhs) used.insert(n->lhs->get_name());
        if (n->copy_from) used.insert(n->copy_from->get_name());
        if (n->copy_to) used.insert(n->copy_to->get_name());
        if (n->target) used.insert(n->target->get_name());
        scan(n->rhs);
        scan(n->predicate);
        for (auto &l : n->lets) scan(l.second);
    });
}

// Runs a compiler with an argument vector (no shell: paths may hold spaces, quotes or `;`).
// The child's stderr goes to `stderr_file` when one is given.  Returns the exit status.
int run(const std::vector<std::string> &argv, const std::string &stderr_file = "") {
    if (debug_level() >= 1) {
        std::cout << "[tiramisu-hip]";
        for (auto &a : argv) std::cout << " " << a;
        std::cout << std::endl;
    }
    std::vector<char *> args;
    for (auto &a : argv) args.push_back(const_cast<char *>(a.c_str()));
    args.push_back(nullptr);
    const pid_t pid = fork();
    if (pid < 0) return -1;
    if (pid == 0) {
        if (!stderr_file.empty()) {
            const int fd = open(stderr_file.c_str(), O_WRONLY | O_CREAT | O_TRUNC, 0644);
            if (fd >= 0) { dup2(fd, 2); close(fd); }
        }
        execvp(args[0], args.data());
        _exit(127);
    }
    int status = 0;
    if (waitpid(pid, &status, 0) < 0) return -1;
    return WIFEXITED(status) ? WEXITSTATUS(status) : -1;
}

// Whitespace-separated words of an option string taken from the environment.
std::vector<std::string> words(const std::string &s) {
    std::vector<std::string> r;
    std::istringstream is(s);
    for (std::string w; is >> w;) r.push_back(w);
    return r;
}

// A path inside a double-quoted string of assembler or C source.
std::string escaped(const std::string &s) {
    std::string r;
    for (char c : s) { if (c == '"' || c == '\\') r += '\\'; r += c; }
    return r;
}

#ifndef TIRAMISU_DEFAULT_HIPCC
#define TIRAMISU_DEFAULT_HIPCC "/opt/rocm/bin/hipcc"
#endif
#ifndef TIRAMISU_DEFAULT_HIP_ARCH
#define TIRAMISU_DEFAULT_HIP_ARCH "gfx950"
#endif

std::string sanitize(const std::string &s) {
    std::string r;
    for (char c : s) r += (isalnum((unsigned char)c) ? c : '_');
    return r;
}

class hip_backend : public backend {
public:
    void generate(function &f, lir::program &prog, const std::string &obj) override {
        context ctx;
        ctx.f = &f;
        ctx.prog = &prog;
        host_gen hg(ctx);

        std::set<std::string> used;
        collect_used_buffers(prog.root, used);
        for (auto &inv : prog.invariants)
            inv.value.visit([&](const expr &x) {
                if (x.get_expr_type() == e_op && x.get_op_type() == o_access) used.insert(x.get_name());
            });

        std::ostringstream body;
        // arguments
        const auto &args = f.get_arguments();
        std::set<std::string> arg_names;
        for (size_t i = 0; i < args.size(); i++) {
            buffer *b = args[i];
            arg_names.insert(b->get_name());
            std::string t = primitive_c_name(b->get_elements_type());
            if (b->get_location() == memory_location::global)
                body << "    " << t << " *" << b->get_name() << " = (" << t << " *)(_a" << i << "->device ? (void *)_a" << i
                     << "->device : (void *)_a" << i << "->host);\n";
            else
                body << "    " << t << " *" << b->get_name() << " = (" << t << " *)_a" << i << "->host;\n";
        }
        // function-wide constants
        for (auto &inv : prog.invariants)
            body << "    const " << primitive_c_name(inv.type) << " " << inv.name << " = " << hg.hp.print(inv.value) << ";\n";
        // temporaries (reference: entry allocation / exit release, tiramisu_codegen_halide.cpp:2488-2530)
        std::vector<std::string> releases;
        for (auto &kv : f.get_buffers()) {
            buffer *b = kv.second;
            if (arg_names.count(b->get_name()) || !used.count(b->get_name())) continue;
            std::string t = primitive_c_name(b->get_elements_type());
            std::string bytes = "(uint64_t)(" + hg.hp.element_count(b) + ") * sizeof(" + t + ")";
            if (b->get_location() == memory_location::global) {
                if (b->get_auto_allocate()) {
                    body << "    " << t << " *" << b->get_name() << " = (" << t << " *)tiramisu_hip_malloc(" << bytes << ");\n";
                    releases.push_back("    tiramisu_hip_free((void *)" + b->get_name() + ");\n");
                } else {
                    body << "    " << t << " *" << b->get_name() << " = nullptr;\n";
                }
            } else if (b->get_location() == memory_location::constant) {
                // its storage is a __constant__ array of the code object; the host only needs its address
                // (the reference's <name>_get_symbol(), tiramisu_codegen_cuda.cpp:817-823)
                if (!b->has_constant_extents()) ERROR("constant-memory buffer " + b->get_name() + " needs constant extents", true);
                ctx.constant_buffers.insert(b->get_name());
                body << "    " << t << " *" << b->get_name() << " = (" << t << " *)tiramisu_hip_module_get_global(_tiramisu_module(), \""
                     << b->get_name() << "\", " << bytes << ");\n";
            } else if (b->get_location() == memory_location::host) {
                if (b->get_auto_allocate()) {
                    body << "    " << t << " *" << b->get_name() << " = (" << t << " *)malloc(" << bytes << ");\n";
                    releases.push_back("    free((void *)" + b->get_name() + ");\n");
                } else {
                    body << "    " << t << " *" << b->get_name() << " = nullptr;\n";
                }
            }
        }
        hg.emit(prog.root, 1);
        body << hg.out.str();
        for (auto it = releases.rbegin(); it != releases.rend(); ++it) body << *it;
        body << "    return 0;\n";

        // ---- kernel file
        const std::string hip_file = obj + ".hip", hsaco = obj + ".hsaco", host_file = obj + ".host.cpp";
        const bool device_code = !ctx.kernels.empty() || !ctx.constant_buffers.empty();
        if (device_code && !std::getenv("HIP_NO_OVERWRITE")) {
            std::ofstream k(hip_file);
            if (!k) ERROR("cannot write " + hip_file, true);
            k << "// Generated by the Tiramisu HIP back-end for gfx950.  Function: " << f.get_name() << "\n";
            k << "#include <hip/hip_runtime.h>\n#include <stdint.h>\n";
            k << ctx.includes;
            std::string all_kernels;
            for (auto &kr : ctx.kernels) all_kernels += kr.source;
            k << c_prelude(true) << c_prelude_opaque(true, all_kernels) << "\n";
            for (auto &nm : ctx.constant_buffers) {
                const buffer *b = f.get_buffers().at(nm);
                long cnt = 1;
                for (auto &d : b->get_dim_sizes()) cnt *= lir::simplify(d).get_int_val();
                if (cnt * (long)primitive_size(b->get_elements_type()) > 65536)
                    ERROR("constant-memory buffer " + nm + " exceeds 64 KiB", true);
                k << "__constant__ " << primitive_c_name(b->get_elements_type()) << " " << nm << "[" << cnt << "];\n";
            }
            for (auto &kr : ctx.kernels) k << "// " << kr.name << ": " << kr.how << "\n" << kr.source << "\n";
        }
        if (device_code) {
            const char *hipcc = std::getenv("HIPCC_PATH");
            const char *arch = backend_option("TIRAMISU_HIP_ARCH");
            const char *flags = backend_option("TIRAMISU_HIP_FLAGS");
            std::vector<std::string> cmd = {hipcc ? hipcc : TIRAMISU_DEFAULT_HIPCC, "--genco",
                                            std::string("--offload-arch=") + (arch ? arch : TIRAMISU_DEFAULT_HIP_ARCH), "-std=c++17"};
            for (auto &w : words(flags ? flags : "-O3")) cmd.push_back(w);
            cmd.push_back("-I" + kernel_dir());            // the kernel headers are included by file name
            for (const char *w : {"-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-o"}) cmd.push_back(w);
            cmd.push_back(hsaco);
            cmd.push_back(hip_file);
            if (run(cmd, obj + ".hipcc.log") != 0) {
                std::ifstream log(obj + ".hipcc.log");
                std::cerr << log.rdbuf();
                ERROR("hipcc failed on " + hip_file, true);
            }
        }
        // ---- host glue
        {
            std::ofstream h(host_file);
            if (!h) ERROR("cannot write " + host_file, true);
            std::string sym = "_tiramisu_hsaco_" + sanitize(f.get_name());
            h << "// Generated by the Tiramisu HIP back-end: host glue of function " << f.get_name() << "\n";
            h << "#include <stdint.h>\n#include <stdlib.h>\n#include <string.h>\n#include <math.h>\n#include <map>\n";
            h << "#include <tiramisu_hip_wrappers.h>\n";
            h << halide_buffer_definition() << c_prelude(false) << c_prelude_opaque(false, body.str()) << "\n";
            for (auto &d : hg.extern_decls) h << d << "\n";
            if (device_code) {
                char *abs_path = realpath(hsaco.c_str(), nullptr);
                const std::string hsaco_abs = abs_path ? abs_path : hsaco;
                free(abs_path);
                h << "__asm__(\".section .rodata\\n.balign 4096\\n.global " << sym << "\\n" << sym << ":\\n.incbin \\\"" << escaped(escaped(hsaco_abs))
                  << "\\\"\\n.global " << sym << "_end\\n" << sym << "_end:\\n.byte 0\\n.previous\\n\");\n";
                h << "extern \"C\" const unsigned char " << sym << "[], " << sym << "_end[];\n";
                h << "static void *_tiramisu_module() {\n    static void *m = tiramisu_hip_module_load((const void *)" << sym
                  << ", (uint64_t)(" << sym << "_end - " << sym << "));\n    return m;\n}\n";
            }
            h << "extern \"C\" int " << f.get_name() << "(";
            for (size_t i = 0; i < args.size(); i++) h << (i ? ", " : "") << "halide_buffer_t *_a" << i;
            h << ")\n{\n" << body.str() << "}\n";
        }
        {
            const char *cxx = std::getenv("TIRAMISU_HOST_CXX");
            const std::string inc = include_dir();
            const std::vector<std::string> cmd = {cxx ? cxx : "g++", "-std=c++17", "-O2", "-fPIC", "-I" + inc, "-c", host_file, "-o", obj};
            if (run(cmd) != 0) ERROR("host compiler failed on " + host_file, true);
        }
        // ---- manifest: what a harness needs to call the function and to know what was emitted
        {
            auto quoted = [](const std::string &t) {
                std::string r = "\"";
                for (char c : t) { if (c == '"' || c == '\\') r += '\\'; r += c; }
                return r + "\"";
            };
            c_printer mp;
            mp.fct = &f;
            std::ofstream m(obj + ".json");
            m << "{\n  \"function\": " << quoted(f.get_name()) << ",\n  \"arguments\": [";
            for (size_t i = 0; i < args.size(); i++) {
                const buffer *b = args[i];
                m << (i ? "," : "") << "\n    {\"name\": " << quoted(b->get_name()) << ", \"type\": " << quoted(primitive_c_name(b->get_elements_type()))
                  << ", \"kind\": " << quoted(b->get_argument_type() == a_input ? "input" : b->get_argument_type() == a_output ? "output" : "temporary")
                  << ", \"memory\": " << quoted(b->get_location() == memory_location::host ? "host" : "device") << ", \"shape\": [";
                for (size_t d = 0; d < b->get_dim_sizes().size(); d++) {
                    const expr e = lir::simplify(b->get_dim_sizes()[d]);
                    m << (d ? ", " : "");
                    if (e.is_integer_literal()) m << e.get_int_val(); else m << quoted(mp.print(e));
                }
                m << "]}";
            }
            m << "\n  ],\n  \"kernel_headers\": " << quoted(device_code ? kernel_dir() : std::string()) << ",\n  \"kernels\": [";
            for (size_t i = 0; i < ctx.kernels.size(); i++)
                m << (i ? "," : "") << "\n    {\"name\": " << quoted(ctx.kernels[i].name) << ", \"how\": " << quoted(ctx.kernels[i].how) << "}";
            m << "\n  ],\n  \"options\": [";
            const auto &opts = f.consulted_backend_options();
            for (size_t i = 0; i < opts.size(); i++)
                m << (i ? "," : "") << "\n    {\"name\": " << quoted(opts[i][0]) << ", \"value\": " << quoted(opts[i][1]) << ", \"from\": " << quoted(opts[i][2]) << "}";
            m << "\n  ]\n}\n";
        }
        for (auto &k : ctx.kernels) f.log(k.name + ": " + k.how);
        if (debug_level() >= 1 || std::getenv("TIRAMISU_HIP_REPORT"))
            for (auto &k : ctx.kernels) std::cout << "[tiramisu-hip] " << f.get_name() << " " << k.name << ": " << k.how << std::endl;
    }
};

struct registrar {
    registrar() { backend::register_backend(hardware_architecture_t::arch_amd_gpu, new hip_backend); }
} the_registrar;

}  // namespace
}  // namespace hipgen
}  // namespace tiramisu
