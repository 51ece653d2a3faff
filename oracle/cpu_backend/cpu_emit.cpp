// PARITY ORACLE -- test infrastructure, not part of the GPU product.
//
// A restatement of the reference's CPU back-end: the same lowered loop program that the HIP
// back-end consumes is printed as C++ with OpenMP, following how the reference turns isl AST
// loops into Halide loops (src/tiramisu_codegen_halide.cpp:2006-2467):
//   * a loop tagged parallel   -> ForType::Parallel  (:2104-2145)  -> #pragma omp parallel for
//   * a loop tagged vectorized -> ForType::Vectorized (:2147-2150) -> #pragma omp simd
//   * a loop tagged unrolled   -> ForType::Unrolled  (:2253-2263)  -> #pragma GCC unroll
//   * GPU-mapped loops         -> plain serial loops (the CPU has no grid)
//   * temporaries              -> heap allocations at entry, released at exit (:2580-2603)
// and compiled for the reference's CPU feature level, AVX + SSE4.1 without FMA
// (:3988-3995): g++ -O2 -mavx -msse4.1 -ffp-contract=off -fopenmp.
//
// Linking this file into a generator registers the arch_cpu back-end, so that
// tiramisu::codegen(args, "f.o") produces host code.  The GPU library never links it.
//
// Parity status: statement order, loop bounds and index expressions come from isl and are
// shared with the GPU path; what this file adds (loop printing, tags) is pinned by
// tests/test_oracle.py against the numpy/C restatements of the reference's wrapper loops.
// Last-ulp float behaviour of Halide/LLVM (their exp/tanh lowering, reassociation under
// vectorize) is not reproducible without the reference's toolchain: parity unpinned for
// that, absorbed by the 1e-4 tolerance.
#include <cstdlib>
#include <fstream>
#include <sstream>

#include <tiramisu/core.h>

#include "../../tiramisu_amd/csrc/c_print.h"
#include "../../tiramisu_amd/csrc/lir.h"

namespace tiramisu {
namespace {

using lir::leaf_kind;
using lir::node_kind;
using lir::node_ptr;

std::string pad(int n) { return std::string(n * 4, ' '); }

struct cpu_gen {
    function *f;
    c_printer cp;
    std::ostringstream out;
    std::set<std::string> declared_in_body;
    std::set<std::string> extern_calls;
    std::vector<std::string> extern_decls;
    int parallel_depth = 0;

    void emit(const node_ptr &n, int ind) {
        if (!n) return;
        switch (n->kind) {
        case node_kind::block:
            for (auto &c : n->children) emit(c, ind);
            break;
        case node_kind::cond:
            out << pad(ind) << "if (" << cp.print(n->condition) << ") {\n";
            emit(n->then_body, ind + 1);
            if (n->else_body) {
                out << pad(ind) << "} else {\n";
                emit(n->else_body, ind + 1);
            }
            out << pad(ind) << "}\n";
            break;
        case node_kind::loop: {
            bool par = n->parallel && parallel_depth == 0;
            if (par) out << pad(ind) << "#pragma omp parallel for schedule(static)\n";
            else if (n->vector_length > 0) out << pad(ind) << "#pragma omp simd\n";
            else if (n->unrolled) out << pad(ind) << "#pragma GCC unroll 16\n";
            out << pad(ind) << "for (int32_t " << n->iterator << " = " << cp.print(n->init) << "; " << n->iterator
                << " <= " << cp.print(n->upper) << "; " << n->iterator << " += " << cp.print(n->increment) << ") {\n";
            if (par) parallel_depth++;
            emit(n->body, ind + 1);
            if (par) parallel_depth--;
            out << pad(ind) << "}\n";
            break;
        }
        case node_kind::leaf: emit_leaf(n, ind); break;
        }
    }

    void emit_leaf(const node_ptr &n, int ind) {
        switch (n->lkind) {
        case leaf_kind::sync: return;
        case leaf_kind::copy: {
            buffer *s = n->copy_from, *d = n->copy_to;
            out << pad(ind) << "memcpy((void *)" << d->get_name() << ", (const void *)" << s->get_name() << ", (size_t)("
                << cp.element_count(s) << ") * sizeof(" << primitive_c_name(s->get_elements_type()) << "));\n";
            return;
        }
        case leaf_kind::allocate: {
            buffer *b = n->target;
            std::string t = primitive_c_name(b->get_elements_type());
            if (b->get_location() == memory_location::reg) {
                out << pad(ind) << t << " " << b->get_name() << " = 0;\n";
            } else if (b->has_constant_extents() && b->get_location() != memory_location::global &&
                       b->get_location() != memory_location::host) {
                out << pad(ind) << t << " " << b->get_name() << "[" << cp.element_count(b) << "];\n";
            } else {
                out << pad(ind) << b->get_name() << " = (" << t << " *)malloc((size_t)(" << cp.element_count(b, n->iterators)
                    << ") * sizeof(" << t << "));\n";
            }
            return;
        }
        case leaf_kind::release:
            if (n->target->get_location() == memory_location::global || n->target->get_location() == memory_location::host)
                out << pad(ind) << "free((void *)" << n->target->get_name() << ");\n";
            return;
        default: break;
        }
        n->rhs.visit([&](const expr &e) {
            if (e.get_expr_type() == e_op && e.get_op_type() == o_call && !extern_calls.count(e.get_name())) {
                extern_calls.insert(e.get_name());
                std::string s = "extern \"C\" " + primitive_c_name(e.get_data_type()) + " " + e.get_name() + "(";
                for (size_t i = 0; i < e.get_arguments().size(); i++) {
                    const expr &a = e.get_arguments()[i];
                    s += (i ? ", " : "") + ((a.get_expr_type() == e_op && a.get_op_type() == o_buffer) ? std::string("void *")
                                             : (a.get_expr_type() == e_op && a.get_op_type() == o_address) ? std::string("halide_buffer_t *")
                                             : primitive_c_name(a.get_data_type()));
                }
                extern_decls.push_back(s + ");");
            }
        });
        if (n->lkind == leaf_kind::let) {
            // a scheduled constant: a scalar visible to the rest of this loop body
            // (reference: LetStmt around the consumer, tiramisu_codegen_halide.cpp:2943-2975)
            out << pad(ind) << "const " << primitive_c_name(n->comp->get_data_type()) << " " << n->comp->get_name() << " = "
                << cp.print(n->rhs) << ";\n";
            return;
        }
        int i2 = ind;
        const bool scoped = !n->lets.empty() || n->predicate.is_defined();
        if (scoped) { out << pad(ind) << "{\n"; i2++; }
        for (auto &l : n->lets)
            out << pad(i2) << "const " << primitive_c_name(l.second.get_data_type()) << " " << l.first << " = " << cp.print(l.second) << ";\n";
        if (n->predicate.is_defined()) { out << pad(i2) << "if (" << cp.print(n->predicate) << ") {\n"; i2++; }
        if (n->lhs) out << pad(i2) << cp.store(n->lhs, n->lhs_index, cp.print(n->rhs), n->rhs.get_data_type()) << "\n";
        else out << pad(i2) << cp.print(n->rhs) << ";\n";
        if (n->predicate.is_defined()) { i2--; out << pad(i2) << "}\n"; }
        if (scoped) out << pad(ind) << "}\n";
    }
};

class cpu_backend : public backend {
public:
    void generate(function &f, lir::program &prog, const std::string &obj) override {
        cpu_gen g;
        g.f = &f;
        g.cp.fct = &f;
        // register buffers that are declared by an allocate leaf are scalars; others are 1-element arrays
        std::set<std::string> leaf_declared, used;
        lir::walk(prog.root, [&](const node_ptr &n) {
            if (n->kind != node_kind::leaf) return;
            if (n->lkind == leaf_kind::allocate) leaf_declared.insert(n->target->get_name());
            auto scan = [&](const expr &e) {
                if (!e.is_defined()) return;
                e.visit([&](const expr &x) {
                    if (x.get_expr_type() == e_op && (x.get_op_type() == o_access || x.get_op_type() == o_buffer)) used.insert(x.get_name());
                });
            };
            if (n->lhs) used.insert(n->lhs->get_name());
            if (n->copy_from) used.insert(n->copy_from->get_name());
            if (n->copy_to) used.insert(n->copy_to->get_name());
            if (n->target) used.insert(n->target->get_name());
            scan(n->rhs); scan(n->predicate);
            for (auto &l : n->lets) scan(l.second);
        });
        for (auto &inv : prog.invariants)
            inv.value.visit([&](const expr &x) { if (x.get_expr_type() == e_op && x.get_op_type() == o_access) used.insert(x.get_name()); });
        g.cp.is_scalar_buffer = [leaf_declared](const buffer *b) {
            return b->get_location() == memory_location::reg && leaf_declared.count(b->get_name()) > 0;
        };

        std::ostringstream body;
        const auto &args = f.get_arguments();
        std::set<std::string> arg_names;
        for (size_t i = 0; i < args.size(); i++) {
            buffer *b = args[i];
            arg_names.insert(b->get_name());
            std::string t = primitive_c_name(b->get_elements_type());
            body << "    " << t << " *" << b->get_name() << " = (" << t << " *)_a" << i << "->host;\n";
        }
        for (auto &inv : prog.invariants)
            body << "    const " << primitive_c_name(inv.type) << " " << inv.name << " = " << g.cp.print(inv.value) << ";\n";
        std::vector<std::string> releases;
        for (auto &kv : f.get_buffers()) {
            buffer *b = kv.second;
            if (arg_names.count(b->get_name()) || !used.count(b->get_name())) continue;
            std::string t = primitive_c_name(b->get_elements_type());
            bool in_body = leaf_declared.count(b->get_name()) > 0;
            bool heap_in_body = in_body && (b->get_location() == memory_location::global || b->get_location() == memory_location::host ||
                                            !b->has_constant_extents());
            if (in_body && !heap_in_body) continue;  // declared where its allocate leaf sits
            if (heap_in_body) {
                body << "    " << t << " *" << b->get_name() << " = nullptr;\n";
            } else {
                body << "    " << t << " *" << b->get_name() << " = (" << t << " *)malloc((size_t)(" << g.cp.element_count(b)
                     << ") * sizeof(" << t << "));\n";
                releases.push_back("    free((void *)" + b->get_name() + ");\n");
            }
        }
        g.emit(prog.root, 1);
        body << g.out.str();
        for (auto it = releases.rbegin(); it != releases.rend(); ++it) body << *it;
        body << "    return 0;\n";

        const std::string src = obj + ".cpu.cpp";
        std::ofstream h(src);
        if (!h) ERROR("cannot write " + src, true);
        h << "// Generated by the CPU back-end restatement (parity oracle). Function: " << f.get_name() << "\n";
        h << "#include <stdint.h>\n#include <stdlib.h>\n#include <string.h>\n#include <math.h>\n";
        h << halide_buffer_definition() << c_prelude(false) << c_prelude_opaque(false, body.str()) << "\n";
        for (auto &d : g.extern_decls) h << d << "\n";
        h << "extern \"C\" int " << f.get_name() << "(";
        for (size_t i = 0; i < args.size(); i++) h << (i ? ", " : "") << "halide_buffer_t *_a" << i;
        h << ")\n{\n" << body.str() << "}\n";
        h.close();
        const char *flags = std::getenv("TIRAMISU_CPU_FLAGS");
        std::string cmd = std::string("g++ -std=c++17 ") + (flags ? flags : "-O2 -mavx -msse4.1 -ffp-contract=off -fopenmp") +
                          " -fPIC -c " + src + " -o " + obj;
        if (std::system(cmd.c_str()) != 0) ERROR("host compiler failed on " + src, true);
    }
};

struct registrar {
    registrar() { backend::register_backend(hardware_architecture_t::arch_cpu, new cpu_backend); }
} the_registrar;

}  // namespace
}  // namespace tiramisu
