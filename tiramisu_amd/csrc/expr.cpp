// Expression trees: construction, type rules, substitution and printing.
// Type rules follow the reference's constructors (include/tiramisu/expr.h:300-520):
// arithmetic keeps the operands' common type, comparisons and logical operators give
// p_boolean, a cast carries its target type.
#include <unordered_map>
#include <tiramisu/core.h>
#include <tiramisu/debug.h>
#include <tiramisu/expr.h>

#include <cmath>
#include <sstream>

namespace tiramisu {

function *global::implicit_fct = nullptr;
primitive_t global::loop_iterator_type = p_int32;
bool global::auto_data_mapping = true;
int var::counter = 0;

void global::set_default_tiramisu_options() {
    loop_iterator_type = p_int32;
    auto_data_mapping = true;
}

int debug_level() {
    static int lvl = [] {
        const char *e = std::getenv("TIRAMISU_DEBUG");
        return e ? std::atoi(e) : 0;
    }();
    return lvl;
}
void str_dump(const std::string &s) { std::cout << s; }
void str_dump(const std::string &s, const char *s2) { std::cout << s << s2; }
void str_dump(const char *s, const char *s2) { std::cout << s << s2; }
void error(const std::string &s, bool exit_program) {
    std::cerr << "Error: " << s << std::endl;
    if (exit_program) std::exit(1);
}

int primitive_size(primitive_t t) {
    switch (t) {
    case p_uint8: case p_int8: case p_boolean: return 1;
    case p_uint16: case p_int16: case p_bfloat16: return 2;
    case p_uint32: case p_int32: case p_float32: return 4;
    case p_uint64: case p_int64: case p_float64: case p_void_ptr: case p_wait_ptr: return 8;
    default: return 0;
    }
}

std::string primitive_c_name(primitive_t t) {
    switch (t) {
    case p_uint8: return "uint8_t";
    case p_uint16: return "uint16_t";
    case p_uint32: return "uint32_t";
    case p_uint64: return "uint64_t";
    case p_int8: return "int8_t";
    case p_int16: return "int16_t";
    case p_int32: return "int32_t";
    case p_int64: return "int64_t";
    case p_float32: return "float";
    case p_float64: return "double";
    case p_boolean: return "bool";
    case p_void_ptr: return "void *";
    case p_bfloat16: return "tiramisu_bf16_t";
    default: return "void";
    }
}

std::string str_from_tiramisu_type_primitive(primitive_t t) {
    switch (t) {
    case p_uint8: return "uint8";
    case p_uint16: return "uint16";
    case p_uint32: return "uint32";
    case p_uint64: return "uint64";
    case p_int8: return "int8";
    case p_int16: return "int16";
    case p_int32: return "int32";
    case p_int64: return "int64";
    case p_float32: return "float32";
    case p_float64: return "float64";
    case p_boolean: return "bool";
    case p_bfloat16: return "bfloat16";
    case p_void_ptr: return "void *";
    default: return "none";
    }
}

bool is_float_type(primitive_t t) { return t == p_float32 || t == p_float64 || t == p_bfloat16; }
bool is_signed_int_type(primitive_t t) {
    return t == p_int8 || t == p_int16 || t == p_int32 || t == p_int64;
}
bool is_int_type(primitive_t t) {
    return is_signed_int_type(t) || t == p_uint8 || t == p_uint16 || t == p_uint32 || t == p_uint64;
}

static bool is_comparison(op_t o) {
    return o == o_eq || o == o_ne || o == o_le || o == o_lt || o == o_ge || o == o_gt;
}

expr::expr(op_t o, expr a) : etype(e_op), op(o), defined(true) {
    dtype = (o == o_logical_not) ? p_boolean : a.get_data_type();
    operands = {a};
}

expr::expr(op_t o, expr a, expr b) : etype(e_op), op(o), defined(true) {
    if (is_comparison(o) || o == o_logical_and || o == o_logical_or)
        dtype = p_boolean;
    else if (o == o_memcpy)
        dtype = p_none;
    else {
        // Literal operands adopt the other side's type so that "x * 2" stays in x's type.
        if (a.get_data_type() != b.get_data_type()) {
            if (b.is_constant() && !a.is_constant())
                b = b.is_integer_literal() && !is_float_type(a.get_data_type())
                        ? value_cast(a.get_data_type(), b.get_int_val())
                        : value_cast(a.get_data_type(), b.get_double_val());
            else if (a.is_constant() && !b.is_constant())
                a = a.is_integer_literal() && !is_float_type(b.get_data_type())
                        ? value_cast(b.get_data_type(), a.get_int_val())
                        : value_cast(b.get_data_type(), a.get_double_val());
        }
        dtype = a.get_data_type();
        if (o == o_right_shift || o == o_left_shift) dtype = a.get_data_type();
    }
    operands = {a, b};
}

expr::expr(op_t o, expr a, expr b, expr c) : etype(e_op), op(o), defined(true) {
    dtype = (o == o_lerp) ? a.get_data_type() : b.get_data_type();
    operands = {a, b, c};
}

expr::expr(op_t o, primitive_t t, expr e) : etype(e_op), op(o), dtype(t), defined(true) {
    if (o != o_cast) ERROR("expr(op, type, expr) expects o_cast", true);
    operands = {e};
}

expr::expr(op_t o, std::string nm) : etype(e_op), op(o), dtype(p_none), defined(true), name(nm) {}

expr::expr(op_t o, std::string nm, std::vector<expr> args, primitive_t t)
    : etype(e_op), op(o), dtype(t), defined(true), name(nm), arguments(std::move(args)) {}

int64_t expr::get_int_val() const {
    if (etype != e_val) ERROR("get_int_val on a non-literal: " + to_str(), true);
    if (is_float_type(dtype)) return (int64_t)val.f64;
    if (is_signed_int_type(dtype)) return val.i64;
    return (int64_t)val.u64;
}

double expr::get_double_val() const {
    if (etype != e_val) ERROR("get_double_val on a non-literal: " + to_str(), true);
    if (is_float_type(dtype)) return val.f64;
    if (is_signed_int_type(dtype)) return (double)val.i64;
    return (double)val.u64;
}

bool expr::is_integer_literal() const { return etype == e_val && !is_float_type(dtype); }

bool expr::is_equal(const expr &e) const {
    if (etype != e.etype || dtype != e.dtype || defined != e.defined) return false;
    if (etype == e_val) return is_float_type(dtype) ? val.f64 == e.val.f64 : val.u64 == e.val.u64;
    if (etype == e_var) return name == e.name;
    if (etype == e_op) {
        if (op != e.op || name != e.name || operands.size() != e.operands.size() ||
            arguments.size() != e.arguments.size())
            return false;
        for (size_t i = 0; i < operands.size(); i++)
            if (!operands[i].is_equal(e.operands[i])) return false;
        for (size_t i = 0; i < arguments.size(); i++)
            if (!arguments[i].is_equal(e.arguments[i])) return false;
    }
    return true;
}

expr expr::substitute(const std::map<std::string, expr> &subs) const {
    return transform([&](const expr &e) -> expr {
        if (e.get_expr_type() == e_var) {
            auto it = subs.find(e.get_name());
            if (it != subs.end()) return it->second;
        }
        return e;
    });
}

expr expr::substitute(const std::vector<std::pair<var, expr>> &subs) const {
    std::map<std::string, expr> m;
    for (auto &p : subs) m[p.first.get_name()] = p.second;
    return substitute(m);
}

expr expr::substitute_access(const std::string &original, const std::string &substitute_name) const {
    return transform([&](const expr &e) -> expr {
        if (e.get_expr_type() == e_op && e.get_op_type() == o_access && e.get_name() == original) {
            expr r = e;
            r.set_name(substitute_name);
            return r;
        }
        return e;
    });
}

expr expr::operator-() const { return expr(o_minus, *this); }
expr expr::operator!() const { return expr(o_logical_not, *this); }

expr value_cast(primitive_t t, double v) {
    switch (t) {
    case p_uint8: return expr((uint8_t)v);
    case p_uint16: return expr((uint16_t)v);
    case p_uint32: return expr((uint32_t)v);
    case p_uint64: return expr((uint64_t)v);
    case p_int8: return expr((int8_t)v);
    case p_int16: return expr((int16_t)v);
    case p_int32: return expr((int32_t)v);
    case p_int64: return expr((int64_t)v);
    case p_float32: return expr((float)v);
    case p_bfloat16: return expr((float)v).copy_with_type(p_bfloat16);
    case p_float64: return expr((double)v);
    case p_boolean: return expr((uint8_t)(v != 0)).copy_with_type(p_boolean);
    default: return expr((double)v);
    }
}

expr value_cast(primitive_t t, int64_t v) {
    switch (t) {
    case p_uint64: return expr((uint64_t)v);
    case p_int64: return expr((int64_t)v);
    case p_none: return expr((int32_t)v);
    default: return value_cast(t, (double)v);
    }
}

expr cast(primitive_t t, const expr &e) {
    if (e.get_data_type() == t) return e;
    return expr(o_cast, t, e);
}

var::var() : var("_v" + std::to_string(counter++)) {}

// Types of the variables declared so far, by name: a later var of the same name takes the declared type
// (reference: var::declared_vars, tiramisu_expr.cpp:88-143; int32 / int64 are interchangeable there too).
static std::unordered_map<std::string, primitive_t> &declared_var_types() {
    static std::unordered_map<std::string, primitive_t> m;
    return m;
}

var::var(std::string nm, bool save) {
    etype = e_var;
    auto d = declared_var_types().find(nm);
    dtype = d != declared_var_types().end() ? d->second : global::get_loop_iterator_data_type();
    defined = true;
    name = nm;
    if (save && d == declared_var_types().end()) declared_var_types()[nm] = dtype;
}

var::var(primitive_t t, std::string nm, bool save) {
    etype = e_var;
    auto d = declared_var_types().find(nm);
    if (d != declared_var_types().end()) {
        const bool ints = (t == p_int32 && d->second == p_int64) || (t == p_int64 && d->second == p_int32);
        if (!ints && d->second != t) ERROR("variable " + nm + " was declared with another type before", true);
        t = d->second;
    }
    dtype = t;
    defined = true;
    name = nm;
    if (save && d == declared_var_types().end()) declared_var_types()[nm] = dtype;
}

var::var(std::string nm, expr lower_bound, expr upper_bound) : var(nm) {
    lower = lower_bound;
    upper = upper_bound;
}

std::string str_tiramisu_type_op(op_t o) {
    switch (o) {
    case o_minus: return "-";
    case o_floor: return "floor";
    case o_sin: return "sin";
    case o_cos: return "cos";
    case o_tan: return "tan";
    case o_asin: return "asin";
    case o_acos: return "acos";
    case o_atan: return "atan";
    case o_sinh: return "sinh";
    case o_cosh: return "cosh";
    case o_tanh: return "tanh";
    case o_asinh: return "asinh";
    case o_acosh: return "acosh";
    case o_atanh: return "atanh";
    case o_abs: return "abs";
    case o_sqrt: return "sqrt";
    case o_expo: return "exp";
    case o_log: return "log";
    case o_ceil: return "ceil";
    case o_round: return "round";
    case o_trunc: return "trunc";
    case o_allocate: return "allocate";
    case o_free: return "free";
    case o_cast: return "cast";
    case o_address: return "address";
    case o_add: return "+";
    case o_sub: return "-";
    case o_mul: return "*";
    case o_div: return "/";
    case o_mod: return "%";
    case o_logical_and: return "&&";
    case o_logical_or: return "||";
    case o_logical_not: return "!";
    case o_eq: return "==";
    case o_ne: return "!=";
    case o_le: return "<=";
    case o_lt: return "<";
    case o_ge: return ">=";
    case o_gt: return ">";
    case o_max: return "max";
    case o_min: return "min";
    case o_right_shift: return ">>";
    case o_left_shift: return "<<";
    case o_memcpy: return "memcpy";
    case o_select: return "select";
    case o_cond: return "cond";
    case o_lerp: return "lerp";
    case o_call: return "call";
    case o_access: return "access";
    case o_address_of: return "address_of";
    case o_lin_index: return "lin_index";
    case o_buffer: return "buffer";
    case o_floordiv: return "floordiv";
    case o_floormod: return "floormod";
    default: return "op?";
    }
}

std::string str_from_tiramisu_type_expr(expr_t t) {
    switch (t) {
    case e_val: return "val";
    case e_var: return "var";
    case e_sync: return "sync";
    case e_op: return "op";
    default: return "none";
    }
}

std::string expr::to_str() const {
    std::ostringstream os;
    if (!defined) return "<undefined>";
    switch (etype) {
    case e_val:
        if (is_float_type(dtype)) os << val.f64;
        else if (is_signed_int_type(dtype)) os << val.i64;
        else os << val.u64;
        break;
    case e_var: os << name; break;
    case e_sync: os << "sync()"; break;
    case e_op:
        if (op == o_access || op == o_call || op == o_address_of || op == o_lin_index) {
            os << name << "(";
            for (size_t i = 0; i < arguments.size(); i++) os << (i ? ", " : "") << arguments[i].to_str();
            os << ")";
        } else if (op == o_allocate || op == o_free || op == o_buffer || op == o_address) {
            os << str_tiramisu_type_op(op) << "(" << name << ")";
        } else if (op == o_cast) {
            os << "cast(" << str_from_tiramisu_type_primitive(dtype) << ", " << operands[0].to_str() << ")";
        } else if (operands.size() == 2 && op >= o_add && op <= o_gt && op != o_logical_not) {
            os << "(" << operands[0].to_str() << " " << str_tiramisu_type_op(op) << " "
               << operands[1].to_str() << ")";
        } else {
            os << str_tiramisu_type_op(op) << "(";
            for (size_t i = 0; i < operands.size(); i++) os << (i ? ", " : "") << operands[i].to_str();
            os << ")";
        }
        break;
    default: os << "<none>";
    }
    return os.str();
}

void expr::dump(bool) const { std::cout << to_str(); }

expr memcpy(const buffer &from, const buffer &to) {
    return expr(o_memcpy, var(p_void_ptr, from.get_name()), var(p_void_ptr, to.get_name()));
}

expr allocate(const buffer &b) { return expr(o_allocate, b.get_name()); }

expr cuda_stream_synchronize() {
    return expr(o_call, "tiramisu_hip_stream_synchronize", {expr((int32_t)0)}, p_int32);
}

expr cublas_gemm(const buffer &A, const buffer &B, buffer &C, expr M, expr N, expr K, expr alpha,
                 expr beta, expr ldA, expr ldB, expr ldC, expr offsetA, expr offsetB, expr offsetC,
                 expr transposeA, expr transposeB) {
    auto u64 = [](expr e) { return e.is_defined() ? cast(p_uint64, e) : expr((uint64_t)0); };
    auto bl = [](expr e) { return e.is_defined() ? cast(p_boolean, e) : value_cast(p_boolean, 0); };
    primitive_t t = A.get_elements_type();
    std::string fn = (t == p_float64) ? "tiramisu_hip_dgemm" : "tiramisu_hip_sgemm";
    return expr(o_call, fn,
                {expr(o_buffer, A.get_name()), expr(o_buffer, B.get_name()), expr(o_buffer, C.get_name()),
                 u64(M), u64(N), u64(K), cast(t, alpha), cast(t, beta), u64(ldA), u64(ldB), u64(ldC),
                 u64(offsetA), u64(offsetB), u64(offsetC), bl(transposeA), bl(transposeB)},
                p_int32);
}

}  // namespace tiramisu
