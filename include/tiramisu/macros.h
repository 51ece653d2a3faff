// Expression helpers that the reference provides as macros (include/tiramisu/macros.h:4-6 of the
// reference: cast, floor, clamp).  Here they are functions of namespace tiramisu -- found by
// argument-dependent lookup wherever an argument is an expr, a var or a constant -- so that they
// do not shadow <cmath>.  cast() itself is declared in expr.h.
#ifndef TIRAMISU_AMD_MACROS_H
#define TIRAMISU_AMD_MACROS_H
#include <tiramisu/expr.h>

namespace tiramisu {

/** Largest integral value not greater than \p e, in e's floating-point type. */
inline expr floor(const expr &e) { return expr(o_floor, e); }

/** \p e limited to [\p min_val, \p max_val]: max(min(e, max_val), min_val), as the reference's macro. */
inline expr clamp(const expr &e, const expr &min_val, const expr &max_val)
{
    return expr(o_max, expr(o_min, e, max_val), min_val);
}

}  // namespace tiramisu
#endif
