// The lowered loop program: what the isl AST of a function becomes before any back-end
// sees it.  Every back-end (HIP kernels + host glue, and the CPU emitter that serves as the
// parity oracle) walks this one tree, so loop structure, leaf order, index expressions and
// predicates are shared by construction.
//
// Expressions are tiramisu::expr with these conventions after lowering:
//   * e_var            loop iterators ("c1", "c3", ...), function-wide constants, let names;
//   * o_access         names a *buffer*, one index expression per buffer dimension;
//   * o_floordiv/mod   floor division / non-negative remainder on signed integers.
#ifndef TIRAMISU_AMD_LIR_H
#define TIRAMISU_AMD_LIR_H
#include <map>
#include <memory>
#include <string>
#include <vector>

#include <tiramisu/core.h>

namespace tiramisu {
namespace lir {

enum class node_kind { block, loop, cond, leaf };
enum class leaf_kind { assign, sync, copy, allocate, release, call, let };   // let: const scalar named after its computation

struct node;
using node_ptr = std::shared_ptr<node>;

struct node {
    node_kind kind = node_kind::block;

    // ---- block ----
    std::vector<node_ptr> children;

    // ---- loop ----
    std::string iterator;     // isl iterator name, "c<2*level+1>"
    int level = -1;           // loop level = index of the dynamic schedule dimension
    expr init;                // first value
    expr upper;               // last value (inclusive)
    expr increment;           // step (1 unless isl strides the loop)
    node_ptr body;
    bool parallel = false;
    int vector_length = 0;
    bool unrolled = false;
    int gpu_block = -1;       // 0/1/2 = blockIdx.x/y/z
    int gpu_thread = -1;      // 0/1/2 = threadIdx.x/y/z

    // ---- cond ----
    expr condition;
    node_ptr then_body, else_body;

    // ---- leaf ----
    leaf_kind lkind = leaf_kind::assign;
    computation *comp = nullptr;
    buffer *lhs = nullptr;              // assign: destination buffer (null for a scalar let)
    std::vector<expr> lhs_index;        // one per dimension of lhs
    expr rhs;                           // assign: value; call: the o_call expression
    expr predicate;                     // undefined when the leaf is unconditional
    std::vector<std::pair<std::string, expr>> lets;  // const scalars declared before the leaf
    buffer *copy_from = nullptr, *copy_to = nullptr; // copy
    buffer *target = nullptr;           // allocate / release
    std::map<std::string, expr> iterators;  // original iterator -> expression of loop iterators
};

struct invariant {
    std::string name;
    primitive_t type;
    expr value;  // lowered: may read argument buffers
};

struct program {
    function *fct = nullptr;
    node_ptr root;
    std::vector<invariant> invariants;
};

/** Linear element offset of \p index in \p b (row-major, last dimension contiguous), with
  * strides cast to the loop iterator type (reference: tiramisu_codegen_halide.cpp:159-214). */
expr linearize(const buffer *b, const std::vector<expr> &index);

/** Fold constants and drop neutral elements; keeps integer semantics exact. */
expr simplify(const expr &e);

/** Visit all nodes, parents first. */
template <typename F> void walk(const node_ptr &n, F &&f) {
    if (!n) return;
    f(n);
    for (auto &c : n->children) walk(c, f);
    walk(n->body, f);
    walk(n->then_body, f);
    walk(n->else_body, f);
}

std::string dump(const node_ptr &n, int indent = 0);

/** Lower computation \p c on its own with the identity schedule.  The result is the loop nest
  * over the computation's iteration-domain dimensions ("c0", "c1", ... outermost first; a
  * dimension with a single value has no loop) with one leaf whose index expressions and value
  * are written in those iterators: the canonical, schedule-independent form that the pattern
  * recognisers analyse.  With \p as_written the value is the computation's expression from before
  * cache_shared() redirected its loads to LDS tiles. */
node_ptr canonical_nest(function &f, computation &c, bool as_written = false);

/** d e / d v for an expression that is affine in variable \p v (other symbols are constants);
  * sets \p ok to false when e is not affine in v. */
expr coefficient(const expr &e, const std::string &v, bool &ok);
bool mentions(const expr &e, const std::string &v);

/** Number of values dimension `d` of `domain` spans from 0: its largest value + 1, as an expression over
  * the domain's parameters (the size of a buffer dimension indexed by that iterator). */
expr extent_of_dimension(function *f, isl_set *domain, int d);

}  // namespace lir
}  // namespace tiramisu
#endif
