// Expression trees of the Tiramisu front-end (reference interface:
// include/tiramisu/expr.h:156-1723).  An expr is a small value type: literals,
// named variables, operators, accesses to computations/buffers and calls.  The same
// type is used after lowering, where an o_access names a *buffer* and carries one
// index per buffer dimension.
#ifndef TIRAMISU_AMD_EXPR_H
#define TIRAMISU_AMD_EXPR_H
#include <cstdint>
#include <map>
#include <string>
#include <type_traits>
#include <utility>
#include <vector>

#include <tiramisu/type.h>

namespace tiramisu {

class function;
class computation;
class buffer;
class var;
class expr;

/** Process-wide settings (reference: expr.h:47-150). */
class global {
    static function *implicit_fct;
    static primitive_t loop_iterator_type;
    static bool auto_data_mapping;
public:
    static function *get_implicit_function() { return implicit_fct; }
    static void set_implicit_function(function *f) { implicit_fct = f; }
    static void set_default_tiramisu_options();
    static void set_loop_iterator_type(primitive_t t) { loop_iterator_type = t; }
    static primitive_t get_loop_iterator_data_type() { return loop_iterator_type; }
    static void set_auto_data_mapping(bool v) { auto_data_mapping = v; }
    static bool is_auto_data_mapping_set() { return auto_data_mapping; }
};

class expr {
protected:
    expr_t etype = e_none;
    op_t op = o_none;
    primitive_t dtype = p_none;
    bool defined = false;
    union {
        uint64_t u64;
        int64_t i64;
        double f64;
    } val{};
    std::string name;
    std::vector<expr> operands;   // operator operands (1..3)
    std::vector<expr> arguments;  // o_access / o_call / o_address_of / o_lin_index arguments

public:
    expr() {}
    /** An undefined expression that only carries a type (used to declare computations
      * whose expression is set later). */
    explicit expr(primitive_t t) : dtype(t) {}

    expr(uint8_t v)  : etype(e_val), dtype(p_uint8),  defined(true) { val.u64 = v; }
    expr(uint16_t v) : etype(e_val), dtype(p_uint16), defined(true) { val.u64 = v; }
    expr(uint32_t v) : etype(e_val), dtype(p_uint32), defined(true) { val.u64 = v; }
    expr(uint64_t v) : etype(e_val), dtype(p_uint64), defined(true) { val.u64 = v; }
    expr(int8_t v)   : etype(e_val), dtype(p_int8),   defined(true) { val.i64 = v; }
    expr(int16_t v)  : etype(e_val), dtype(p_int16),  defined(true) { val.i64 = v; }
    expr(int32_t v)  : etype(e_val), dtype(p_int32),  defined(true) { val.i64 = v; }
    expr(int64_t v)  : etype(e_val), dtype(p_int64),  defined(true) { val.i64 = v; }
    expr(float v)    : etype(e_val), dtype(p_float32), defined(true) { val.f64 = v; }
    expr(double v)   : etype(e_val), dtype(p_float64), defined(true) { val.f64 = v; }

    /** Unary operator (o_minus, o_floor, o_tanh, o_expo, o_logical_not, ...). */
    expr(op_t o, expr a);
    /** Binary operator. */
    expr(op_t o, expr a, expr b);
    /** Ternary operator (o_select, o_cond, o_lerp). */
    expr(op_t o, expr a, expr b, expr c);
    /** Cast of \p e to type \p t (o must be o_cast). */
    expr(op_t o, primitive_t t, expr e);
    /** o_allocate / o_free / o_address / o_buffer of the buffer called \p nm. */
    expr(op_t o, std::string nm);
    /** o_access / o_call / o_address_of / o_lin_index with an argument list. */
    expr(op_t o, std::string nm, std::vector<expr> args, primitive_t t);

    bool is_defined() const { return defined; }
    expr_t get_expr_type() const { return etype; }
    op_t get_op_type() const { return op; }
    primitive_t get_data_type() const { return dtype; }
    const std::string &get_name() const { return name; }
    void set_name(const std::string &n) { name = n; }
    int get_n_arg() const { return (int)operands.size(); }
    const expr &get_operand(int i) const { return operands.at(i); }
    const std::vector<expr> &get_operands() const { return operands; }
    const std::vector<expr> &get_access() const { return arguments; }
    const std::vector<expr> &get_arguments() const { return arguments; }
    int get_n_dim_access() const { return (int)arguments.size(); }
    void set_access(std::vector<expr> a) { arguments = std::move(a); }

    int64_t get_int_val() const;
    double get_double_val() const;
    uint8_t get_uint8_value() const { return (uint8_t)val.u64; }
    int32_t get_int32_value() const { return (int32_t)val.i64; }
    float get_float32_value() const { return (float)val.f64; }
    double get_float64_value() const { return val.f64; }
    /** True for literals. */
    bool is_constant() const { return etype == e_val; }
    bool is_integer_literal() const;
    /** Structural equality. */
    bool is_equal(const expr &e) const;

    /** Replace variables by expressions (matched by name). */
    expr substitute(const std::vector<std::pair<var, expr>> &subs) const;
    expr substitute(const std::map<std::string, expr> &subs) const;
    /** Rewrite every o_access to \p original so that it targets \p substitute. */
    expr substitute_access(const std::string &original, const std::string &substitute) const;
    /** Apply \p f bottom-up to every node and return the rebuilt tree. */
    template <typename F> expr transform(F &&f) const {
        expr r = *this;
        for (auto &o : r.operands) o = o.transform(f);
        for (auto &a : r.arguments) a = a.transform(f);
        return f(r);
    }
    /** Visit every node (pre-order). */
    template <typename F> void visit(F &&f) const {
        f(*this);
        for (auto &o : operands) o.visit(f);
        for (auto &a : arguments) a.visit(f);
    }

    std::string to_str() const;
    void dump(bool exhaustive = false) const;

    expr operator-() const;
    expr operator!() const;
    /** Copy with a different data type (no conversion node). */
    expr copy_with_type(primitive_t t) const { expr e = *this; e.dtype = t; return e; }
};

/** A literal of type \p t holding \p v converted to that type (reference: expr.h value_cast). */
expr value_cast(primitive_t t, double v);
expr value_cast(primitive_t t, int64_t v);
inline expr value_cast(primitive_t t, int v) { return value_cast(t, (int64_t)v); }
inline expr value_cast(primitive_t t, float v) { return value_cast(t, (double)v); }
/** \p e converted to \p t; a no-op if it already has that type. */
expr cast(primitive_t t, const expr &e);

class var : public expr {
    expr lower, upper;
    static int counter;
public:
    var();
    var(std::string nm, bool save = true);
    var(primitive_t t, std::string nm, bool save = true);
    var(std::string nm, expr lower_bound, expr upper_bound);
    const expr &get_lower() const { return lower; }
    const expr &get_upper() const { return upper; }
};

/** Barrier between the threads of a GPU block (reference: expr.h:1713-1723). */
class sync : public expr {
public:
    sync() { etype = e_sync; dtype = p_none; defined = true; }
};

#define TIRAMISU_BINOP(sym, code)                                                          \
    inline expr operator sym(const expr &a, const expr &b) { return expr(code, a, b); }    \
    template <typename T, typename std::enable_if<std::is_arithmetic<T>::value, int>::type = 0> \
    expr operator sym(const expr &a, T b) {                                                \
        return expr(code, a, std::is_floating_point<T>::value                               \
                                 ? value_cast(a.get_data_type(), (double)b)                \
                                 : value_cast(a.get_data_type(), (int64_t)b));             \
    }                                                                                      \
    template <typename T, typename std::enable_if<std::is_arithmetic<T>::value, int>::type = 0> \
    expr operator sym(T a, const expr &b) {                                                \
        return expr(code, std::is_floating_point<T>::value                                 \
                              ? value_cast(b.get_data_type(), (double)a)                   \
                              : value_cast(b.get_data_type(), (int64_t)a), b);             \
    }
TIRAMISU_BINOP(+, o_add)
TIRAMISU_BINOP(-, o_sub)
TIRAMISU_BINOP(*, o_mul)
TIRAMISU_BINOP(/, o_div)
TIRAMISU_BINOP(%, o_mod)
TIRAMISU_BINOP(>>, o_right_shift)
TIRAMISU_BINOP(<<, o_left_shift)
TIRAMISU_BINOP(&&, o_logical_and)
TIRAMISU_BINOP(||, o_logical_or)
TIRAMISU_BINOP(==, o_eq)
TIRAMISU_BINOP(!=, o_ne)
TIRAMISU_BINOP(<, o_lt)
TIRAMISU_BINOP(<=, o_le)
TIRAMISU_BINOP(>, o_gt)
TIRAMISU_BINOP(>=, o_ge)
#undef TIRAMISU_BINOP

/** Whole-buffer copy between a host buffer and a GPU buffer, in either direction
  * (reference: tiramisu_expr.cpp:186-196). */
expr memcpy(const buffer &from, const buffer &to);
/** Declaration (shared/local/register) or device allocation (global) of \p b at the
  * point where the computation holding this expression is scheduled. */
expr allocate(const buffer &b);
/** Wait for the work queued on the calling thread's stream. */
expr cuda_stream_synchronize();
inline expr hip_stream_synchronize() { return cuda_stream_synchronize(); }
/** Row-major GEMM library call C = alpha*op(A)*op(B) + beta*C on GPU buffers; lowered to this
  * back-end's own MFMA kernel (reference: tiramisu_expr.cpp:198-242). */
expr cublas_gemm(const buffer &A, const buffer &B, buffer &C, expr M, expr N, expr K,
                 expr alpha, expr beta, expr ldA = expr(), expr ldB = expr(), expr ldC = expr(),
                 expr offsetA = expr(), expr offsetB = expr(), expr offsetC = expr(),
                 expr transposeA = expr(), expr transposeB = expr());

std::string str_from_tiramisu_type_expr(expr_t t);
std::string str_tiramisu_type_op(op_t o);

}  // namespace tiramisu
#endif
