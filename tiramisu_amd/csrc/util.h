// Small string helpers shared by the compiler sources.
#ifndef TIRAMISU_AMD_UTIL_H
#define TIRAMISU_AMD_UTIL_H
#include <string>
#include <vector>

namespace tiramisu {

inline std::string join(const std::vector<std::string> &v, const std::string &sep) {
    std::string r;
    for (size_t i = 0; i < v.size(); i++) r += (i ? sep : std::string()) + v[i];
    return r;
}

inline std::string replace_all(std::string s, const std::string &from, const std::string &to) {
    size_t pos = 0;
    while ((pos = s.find(from, pos)) != std::string::npos) {
        s.replace(pos, from.size(), to);
        pos += to.size();
    }
    return s;
}

class expr;
/** isl syntax for an integer (quasi-)affine expression; sets \p ok to false otherwise. */
std::string expr_to_isl_str(const expr &e, bool &ok);

/** skew(i, j, a, b): divides a and b by their common divisor and completes (a, b) to a matrix of determinant 1
  * with the second row (gamma, sigma) that computation::skew uses; false when a < 0, b == 0 or none is found. */
bool skewing_second_row(int &a, int &b, int &gamma, int &sigma);

class computation;
/** { consumer[iterators] -> producer[indices] } for every read of \p producer in the consumer's expression and
  * predicate, over the consumer's iteration domain (and, on request, inside the producer's); null if none.  An index
  * that is not affine is an error, or -- with \p any_where_not_affine -- a dimension left free (the read may be of any element). */
struct isl_map *reads_of(computation &consumer, computation &producer, bool within_producer_domain = true,
                         bool any_where_not_affine = false);

}  // namespace tiramisu
#endif
