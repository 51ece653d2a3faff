// C++ wrapper of taps_in_constant_memory (tests/programs/taps_in_constant_memory.cpp): host
// buffers in and out, the generated function does every copy itself.  Same style as the
// reference's wrappers (Halide::Buffer, nested-loop reference, compare_buffers).
// links: tests/programs/build/taps_in_constant_memory.o
#include "Halide.h"
#include <tiramisu/utils.h>

#include <cstdlib>

extern "C" int taps_in_constant_memory(halide_buffer_t *image, halide_buffer_t *taps, halide_buffer_t *filtered);

int main(int, char **)
{
    const int ROWS = 70, COLS = 100, TAPS = 5;
    Halide::Buffer<float> image(COLS, ROWS), taps(TAPS), filtered(COLS - TAPS + 1, ROWS), expected(COLS - TAPS + 1, ROWS);
    std::srand(61);
    for (int r = 0; r < ROWS; r++)
        for (int c = 0; c < COLS; c++) image(c, r) = (float)(std::rand() % 10 - 5);
    for (int t = 0; t < TAPS; t++) taps(t) = (float)(std::rand() % 7 - 3);
    init_buffer(filtered, -1.0f);
    for (int r = 0; r < ROWS; r++)
        for (int c = 0; c + TAPS <= COLS; c++) {
            float acc = image(c, r) * taps(0);
            for (int t = 1; t < TAPS; t++) acc += image(c + t, r) * taps(t);
            expected(c, r) = acc;
        }

    taps_in_constant_memory(image.raw_buffer(), taps.raw_buffer(), filtered.raw_buffer());
    compare_buffers("taps_in_constant_memory", filtered, expected);
    return 0;
}
