// Pattern-directed kernel emitters (placeholders until the recognisers are filled in).
#include "hip_backend.h"

namespace tiramisu {
namespace hipgen {

bool emit_contraction(context &, const lir::node_ptr &, launch_plan &) { return false; }
bool emit_stencil(context &, const lir::node_ptr &, const lir::node_ptr &, launch_plan &) { return false; }

}  // namespace hipgen
}  // namespace tiramisu
