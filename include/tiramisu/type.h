// Enumerations of the Tiramisu front-end: expression kinds, primitive types, operators,
// argument kinds and code-generation targets.  The enumerator names are the public
// vocabulary of Tiramisu programs (reference: include/tiramisu/type.h:14-164); this
// build adds p_bfloat16 (bf16 storage for the MFMA contraction variant) and the
// arch_amd_gpu target, and has no Halide conversions.
#ifndef TIRAMISU_AMD_TYPE_H
#define TIRAMISU_AMD_TYPE_H
#include <cstdint>
#include <string>

namespace tiramisu {

enum expr_t { e_val, e_var, e_sync, e_op, e_none };

enum primitive_t {
    p_uint8, p_uint16, p_uint32, p_uint64, p_int8, p_int16, p_int32, p_int64,
    p_float32, p_float64, p_boolean, p_async, p_wait_ptr, p_void_ptr, p_none,
    p_bfloat16  // storage-only 16-bit brain float; arithmetic is carried out in fp32
};

enum op_t {
    // unary
    o_minus, o_floor, o_sin, o_cos, o_tan, o_asin, o_acos, o_atan, o_sinh, o_cosh, o_tanh,
    o_asinh, o_acosh, o_atanh, o_abs, o_sqrt, o_expo, o_log, o_ceil, o_round, o_trunc,
    o_allocate, o_free, o_cast, o_address,
    // binary
    o_add, o_sub, o_mul, o_div, o_mod, o_logical_and, o_logical_or, o_logical_not,
    o_eq, o_ne, o_le, o_lt, o_ge, o_gt, o_max, o_min, o_right_shift, o_left_shift, o_memcpy,
    // ternary
    o_select, o_cond, o_lerp,
    // name + argument list
    o_call, o_access, o_address_of, o_lin_index, o_type, o_dummy, o_buffer,
    o_none,
    // lowering-only operators produced by the AST layer: floor division and the
    // matching non-negative remainder on signed integers
    o_floordiv, o_floormod
};

enum argument_t { a_input, a_output, a_temporary };

enum class rank_t { r_sender, r_receiver };

enum class hardware_architecture_t {
    arch_cpu,
    arch_nvidia_gpu,   // kept so that existing programs compile; selects the configured GPU back-end
    arch_flexnlp,      // not provided
    arch_amd_gpu       // HIP / gfx950 back-end
};

/** Size in bytes of one element of type \p t. */
int primitive_size(primitive_t t);
/** C spelling of \p t as used by the emitters ("float", "int32_t", ...). */
std::string primitive_c_name(primitive_t t);
std::string str_from_tiramisu_type_primitive(primitive_t t);
bool is_float_type(primitive_t t);
bool is_signed_int_type(primitive_t t);
bool is_int_type(primitive_t t);

}  // namespace tiramisu
#endif
