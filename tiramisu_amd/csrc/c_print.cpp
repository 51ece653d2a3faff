#include "c_print.h"

#include <cmath>
#include <cstdio>
#include <sstream>

#include "lir.h"

namespace tiramisu {

std::string c_printer::literal(const expr &e) const {
    char buf[64];
    primitive_t t = e.get_data_type();
    if (t == p_float32 || t == p_bfloat16) {
        double v = e.get_double_val();
        if (std::isinf(v)) return v > 0 ? "INFINITY" : "(-INFINITY)";
        if (std::isnan(v)) return "NAN";
        snprintf(buf, sizeof buf, "%.9g", v);
        std::string s = buf;
        if (s.find_first_of(".en") == std::string::npos) s += ".0";
        s += "f";
        return v < 0 ? "(" + s + ")" : s;
    }
    if (t == p_float64) {
        double v = e.get_double_val();
        snprintf(buf, sizeof buf, "%.17g", v);
        std::string s = buf;
        if (s.find_first_of(".en") == std::string::npos) s += ".0";
        return v < 0 ? "(" + s + ")" : s;
    }
    if (t == p_boolean) return e.get_int_val() ? "true" : "false";
    int64_t v = e.get_int_val();
    std::string s = std::to_string(v);
    if (t == p_int64) s += "ll";
    else if (t == p_uint64) s += "ull";
    else if (t == p_uint32) s += "u";
    else if (t == p_uint8 || t == p_uint16 || t == p_int8 || t == p_int16) s = "((" + primitive_c_name(t) + ")" + s + ")";
    return v < 0 ? "(" + s + ")" : s;
}

static const char *math_name(op_t o) {
    switch (o) {
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
    case o_sqrt: return "sqrt";
    case o_expo: return "exp";
    case o_log: return "log";
    case o_ceil: return "ceil";
    case o_round: return "round";
    case o_trunc: return "trunc";
    default: return nullptr;
    }
}

std::string c_printer::element(const buffer *b, const std::vector<expr> &index) const {
    if (used_buffers) used_buffers->insert(b->get_name());
    if (is_scalar_buffer(b)) return b->get_name();
    // indices are linearised in the 32-bit loop iterator type (the reference's, expr.h:130-143)
    if (b->has_constant_extents()) {
        double cnt = 1;
        for (auto &d : b->get_dim_sizes()) cnt *= (double)lir::simplify(d).get_int_val();
        if (cnt > 2147483647.0)
            ERROR("buffer " + b->get_name() + " holds more than 2^31-1 elements: its 32-bit linear index would wrap", true);
    }
    return b->get_name() + "[" + print(lir::linearize(b, index)) + "]";
}

std::string c_printer::store(const buffer *b, const std::vector<expr> &index, const std::string &value,
                             primitive_t value_type) const {
    std::string v = value;
    primitive_t bt = b->get_elements_type();
    if (bt == p_bfloat16) v = "t_f32_to_bf16(" + v + ")";
    else if (bt != value_type && value_type != p_none) v = "(" + primitive_c_name(bt) + ")(" + v + ")";
    if (device && streaming_stores && streaming_stores->count(b->get_name()))
        return "__builtin_nontemporal_store((" + primitive_c_name(bt == p_bfloat16 ? p_uint16 : bt) + ")(" + v + "), &" + element(b, index) + ");";
    return element(b, index) + " = " + v + ";";
}

std::string c_printer::element_count(const buffer *b) const {
    return element_count(b, {});
}

// extents of a buffer allocated inside a loop nest may name the allocating computation's iterators
// (f_b[i + 1] allocated at loop i): they are written in the loop iterators of the generated code
std::string c_printer::element_count(const buffer *b, const std::map<std::string, expr> &iterators) const {
    expr n;
    for (auto &d0 : b->get_dim_sizes()) {
        const expr d = iterators.empty() ? d0 : lir::simplify(d0.substitute(iterators));
        n = n.is_defined() ? lir::simplify(n * cast(p_int64, d)) : cast(p_int64, d);
    }
    return n.is_defined() ? print(n) : "1";
}

std::string c_printer::print(const expr &e) const {
    if (!e.is_defined()) ERROR("printing an undefined expression", true);
    switch (e.get_expr_type()) {
    case e_val: return literal(e);
    case e_var:
        if (used_scalars) used_scalars->insert(e.get_name());
        return e.get_name();
    case e_op: break;
    default: ERROR("cannot print expression " + e.to_str(), true);
    }
    op_t o = e.get_op_type();
    primitive_t t = e.get_data_type();
    auto P = [&](int i) { return print(e.get_operand(i)); };
    // C promotes 8- and 16-bit integers to int; the reference's expressions keep their type and wrap
    // (uint8 + uint8 is a uint8), so arithmetic on narrow types is cast back after every operation
    const bool narrow = t == p_uint8 || t == p_int8 || t == p_uint16 || t == p_int16;
    auto keep = [&](const std::string &v) { return narrow ? "((" + primitive_c_name(t) + ")" + v + ")" : v; };
    auto bin = [&](const char *sym) { return "(" + P(0) + " " + sym + " " + P(1) + ")"; };
    // hipcc 7.2 for gfx950 has been seen to compute (int8_t)((int8_t)(a * b) / 2) wrongly (x + 3 instead of x / 2 for
    // most inputs; gcc and the host side of the same clang are right): the truncation of a signed narrow product is
    // folded into a following operation that depends on its sign.  The products of signed 8- and 16-bit values, and
    // the left operands of their /, % and >>, therefore pass through t_opaque(): on the device an empty asm statement
    // that hands the sign-extended value back as one the optimiser knows nothing about, on the host the identity.
    const bool narrow_signed = t == p_int8 || t == p_int16;
    auto bin_opaque_left = [&](const char *sym) { return "(t_opaque(" + P(0) + ") " + sym + " " + P(1) + ")"; };
    if (const char *m = math_name(o)) {
        std::string fn = m;
        if (t == p_float32 || t == p_bfloat16) fn += "f";
        return fn + "(" + P(0) + ")";
    }
    switch (o) {
    case o_minus: return keep("(-" + P(0) + ")");
    case o_abs: return (is_float_type(t) ? (t == p_float64 ? "fabs(" : "fabsf(") : "t_abs(") + P(0) + ")";
    case o_logical_not: return "(!" + P(0) + ")";
    case o_cast:
        if (t == p_bfloat16) return "t_bf16_to_f32(t_f32_to_bf16(" + P(0) + "))";
        return "((" + primitive_c_name(t) + ")(" + P(0) + "))";
    case o_add: return keep(bin("+"));
    case o_sub: return keep(bin("-"));
    case o_mul: return narrow_signed ? "t_opaque(" + keep(bin("*")) + ")" : keep(bin("*"));
    case o_div: return keep(narrow_signed ? bin_opaque_left("/") : bin("/"));
    case o_mod: return is_float_type(t) ? "fmod(" + P(0) + ", " + P(1) + ")" : keep(narrow_signed ? bin_opaque_left("%") : bin("%"));
    case o_floordiv: return "t_floordiv(" + P(0) + ", " + P(1) + ")";
    case o_floormod: return "t_floormod(" + P(0) + ", " + P(1) + ")";
    case o_logical_and: return bin("&&");
    case o_logical_or: return bin("||");
    case o_eq: return bin("==");
    case o_ne: return bin("!=");
    case o_le: return bin("<=");
    case o_lt: return bin("<");
    case o_ge: return bin(">=");
    case o_gt: return bin(">");
    case o_max: return "t_max(" + P(0) + ", " + P(1) + ")";
    case o_min: return "t_min(" + P(0) + ", " + P(1) + ")";
    case o_right_shift: return keep(narrow_signed ? bin_opaque_left(">>") : bin(">>"));
    case o_left_shift: return keep(bin("<<"));
    case o_select: case o_cond: return "(" + P(0) + " ? " + P(1) + " : " + P(2) + ")";
    case o_lerp: return "t_lerp(" + P(0) + ", " + P(1) + ", " + P(2) + ")";
    case o_access: {
        auto it = fct->get_buffers().find(e.get_name());
        if (it == fct->get_buffers().end()) {
            // an access to a computation outside a loop nest (the size of a buffer read from an input, as in
            // S0_b({N_input(0), N_input(0)})): the element of the computation's buffer, for one-to-one mappings
            for (computation *c : fct->get_computations())
                if (c->get_name() == e.get_name() && c->get_buffer() && (int)e.get_access().size() == c->get_buffer()->get_n_dims())
                    return element(c->get_buffer(), e.get_access());
            ERROR("access to unknown buffer " + e.get_name(), true);
        }
        std::string s = element(it->second, e.get_access());
        if (it->second->get_elements_type() == p_bfloat16) s = "t_bf16_to_f32(" + s + ")";
        return s;
    }
    case o_buffer: {
        if (used_buffers) used_buffers->insert(e.get_name());
        return e.get_name();
    }
    case o_address: {
        // the halide_buffer_t of an argument buffer: generated host functions name their arguments _a0, _a1, ...
        const std::string &nm = e.get_operand(0).get_name();
        if (device) ERROR("address of buffer " + nm + " inside a GPU kernel", true);
        if (used_buffers) used_buffers->insert(nm);
        const auto &args = fct->get_arguments();
        for (size_t i = 0; i < args.size(); i++)
            if (args[i]->get_name() == nm) return "_a" + std::to_string(i);
        ERROR("address of buffer " + nm + ", which is not an argument of the function (only arguments have a halide_buffer_t)", true);
    }
    case o_address_of: {
        auto it = fct->get_buffers().find(e.get_name());
        if (it == fct->get_buffers().end()) ERROR("address of unknown buffer " + e.get_name(), true);
        return "(&" + element(it->second, e.get_access()) + ")";
    }
    case o_call: {
        std::string s = e.get_name() + "(";
        for (size_t i = 0; i < e.get_arguments().size(); i++) s += (i ? ", " : "") + print(e.get_arguments()[i]);
        return s + ")";
    }
    default: ERROR("cannot print operator " + str_tiramisu_type_op(o), true);
    }
    return "";
}

std::string c_prelude(bool device) {
    std::string q = device ? "__device__ __forceinline__" : "static inline";
    std::ostringstream os;
    os << "typedef uint16_t tiramisu_bf16_t;\n";
    os << "template <typename T> " << q << " T t_max(T a, T b) { return a > b ? a : b; }\n";
    os << "template <typename T> " << q << " T t_min(T a, T b) { return a < b ? a : b; }\n";
    os << "template <typename T> " << q << " T t_abs(T a) { return a < 0 ? -a : a; }\n";
    // lerp as the reference's CPU back-end (Halide) defines it: a (1 - w) + b w, an unsigned integer
    // weight standing for w / (largest value of its type), rounded to nearest
    os << "template <typename T> " << q << " T t_lerp(T a, T b, T w) { return a * (1 - w) + b * w; }\n";
    os << q << " uint8_t t_lerp(uint8_t a, uint8_t b, uint8_t w) { return (uint8_t)(((uint32_t)a * (255u - w) + (uint32_t)b * w + 127u) / 255u); }\n";
    os << q << " uint16_t t_lerp(uint16_t a, uint16_t b, uint16_t w) { return (uint16_t)(((uint64_t)a * (65535u - w) + (uint64_t)b * w + 32767u) / 65535u); }\n";
    // floor division and the remainder with the sign of the divisor's magnitude (Euclidean for
    // positive divisors): what the CPU back-end of the reference computes for integer / and %
    os << "template <typename T> " << q << " T t_floordiv(T a, T b) { T q = a / b; T r = a % b; "
          "return (r != 0 && ((r < 0) != (b < 0))) ? q - 1 : q; }\n";
    os << "template <typename T> " << q << " T t_floormod(T a, T b) { T r = a % b; "
          "return (r != 0 && ((r < 0) != (b < 0))) ? r + b : r; }\n";
    os << q << " float t_bf16_to_f32(tiramisu_bf16_t v) { union { uint32_t u; float f; } x; x.u = ((uint32_t)v) << 16; return x.f; }\n";
    os << q << " tiramisu_bf16_t t_f32_to_bf16(float f) { union { uint32_t u; float f; } x; x.f = f; "
          "if ((x.u & 0x7fffffffu) > 0x7f800000u) return (tiramisu_bf16_t)((x.u >> 16) | 0x40); "
          "uint32_t r = 0x7fffu + ((x.u >> 16) & 1u); return (tiramisu_bf16_t)((x.u + r) >> 16); }\n";
    return os.str();
}

// t_opaque (see c_printer::print), added to a generated file whose code uses it
std::string c_prelude_opaque(bool device, const std::string &code) {
    if (code.find("t_opaque(") == std::string::npos) return "";
    if (device)
        return "template <typename T> __device__ __forceinline__ T t_opaque(T v) { int32_t w = v; asm(\"\" : \"+v\"(w)); return (T)w; }\n";
    return "template <typename T> static inline T t_opaque(T v) { return v; }\n";
}

std::string halide_buffer_definition() {
    return R"(#ifndef HALIDE_HALIDERUNTIME_H
typedef struct halide_dimension_t { int32_t min, extent, stride; uint32_t flags; } halide_dimension_t;
struct halide_type_t { uint8_t code; uint8_t bits; uint16_t lanes; };
typedef struct halide_buffer_t {
    uint64_t device;
    const struct halide_device_interface_t *device_interface;
    uint8_t *host;
    uint64_t flags;
    struct halide_type_t type;
    int32_t dimensions;
    halide_dimension_t *dim;
    void *padding;
} halide_buffer_t;
#endif
)";
}

}  // namespace tiramisu
