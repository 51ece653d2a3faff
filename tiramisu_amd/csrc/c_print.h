// Printing of lowered expressions as C/C++/HIP source text.  Used by the HIP kernel emitter,
// by the host-glue emitter and by the CPU emitter that serves as the parity oracle, so the
// three agree on the meaning of every operator by construction.
#ifndef TIRAMISU_AMD_C_PRINT_H
#define TIRAMISU_AMD_C_PRINT_H
#include <map>
#include <functional>
#include <set>
#include <string>

#include <tiramisu/core.h>

namespace tiramisu {

struct c_printer {
    function *fct = nullptr;
    /** true inside HIP device code (selects device spellings of helpers). */
    bool device = false;
    /** Buffers whose name alone denotes the value (register buffers). */
    std::function<bool(const buffer *)> is_scalar_buffer = [](const buffer *b) {
        return b->get_location() == memory_location::reg;
    };
    /** Records every buffer and free variable printed (for kernel parameter discovery). */
    std::set<std::string> *used_buffers = nullptr;
    std::set<std::string> *used_scalars = nullptr;
    /** Device code: buffers whose stores carry the non-temporal hint (written and never read by the kernel). */
    const std::set<std::string> *streaming_stores = nullptr;

    std::string print(const expr &e) const;
    /** "buf[linear index]" or the bare name for register buffers. */
    std::string element(const buffer *b, const std::vector<expr> &index) const;
    /** Text of a store of \p value (already printed, in the computation's type) to an element. */
    std::string store(const buffer *b, const std::vector<expr> &index, const std::string &value,
                      primitive_t value_type) const;
    std::string literal(const expr &e) const;
    /** Number of elements of \p b as an expression text. */
    std::string element_count(const buffer *b) const;
    std::string element_count(const buffer *b, const std::map<std::string, expr> &iterators) const;
};

/** Helper functions (floor division, min/max, bf16 conversion) that printed code relies on;
  * \p device selects __device__ qualifiers. */
std::string c_prelude(bool device);
std::string c_prelude_opaque(bool device, const std::string &code);
/** Layout-compatible definition of halide_buffer_t for generated host code. */
std::string halide_buffer_definition();

}  // namespace tiramisu
#endif
