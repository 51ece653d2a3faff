// Generators of the reference's image benchmarks include Halide's image I/O helpers although only
// their wrappers load images (benchmarks/halide/*_tiramisu.cpp).  Nothing of it is needed to
// generate code; wrappers that want image files bring their own loader.
#ifndef TIRAMISU_AMD_HALIDE_IMAGE_IO_SHIM_H
#define TIRAMISU_AMD_HALIDE_IMAGE_IO_SHIM_H
#include "Halide.h"
#endif
