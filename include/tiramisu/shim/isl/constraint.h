// Tiramisu programs written for the reference include isl's headers out of habit; the ROCm image
// ships libisl without them.  Every <isl/...> name in this directory resolves to the declarations
// this build uses itself (tiramisu/isl_api.h).
#include <tiramisu/isl_api.h>
