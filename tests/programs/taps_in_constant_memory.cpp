// A 5-tap horizontal filter whose taps live in GPU constant memory, with all CPU<->GPU copies
// inserted by codegen(): every GPU buffer names its CPU counterpart (last constructor argument),
// so the inputs are copied in before the first computation -- the taps with a copy to the constant
// symbol -- and the output is copied back after the last one.  Same features as the reference's
// benchmarks/halide/gaussiangpu_tiramisu.cpp:61-79 (tag_gpu_constant weights) and its automatic
// communication (src/tiramisu_function.cpp:379-435), on a program of its own.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

int main()
{
    const int ROWS = 70, COLS = 100, TAPS = 5;
    tiramisu::init("taps_in_constant_memory");
    function *fct = global::get_implicit_function();

    var r("r", 0, ROWS), c("c", 0, COLS - TAPS + 1), cc("cc", 0, COLS), t("t", 0, TAPS);
    var rb("rb"), rt("rt"), cb("cb"), ct("ct");

    buffer image("image", {ROWS, COLS}, p_float32, a_input);
    buffer taps("taps", {TAPS}, p_float32, a_input);
    buffer filtered("filtered", {ROWS, COLS - TAPS + 1}, p_float32, a_output);

    buffer image_gpu("image_gpu", {ROWS, COLS}, p_float32, a_temporary, fct, "image");
    buffer taps_gpu("taps_gpu", {TAPS}, p_float32, a_temporary, fct, "taps");
    buffer filtered_gpu("filtered_gpu", {ROWS, COLS - TAPS + 1}, p_float32, a_temporary, fct, "filtered");
    image_gpu.tag_gpu_global();
    taps_gpu.tag_gpu_constant();
    filtered_gpu.tag_gpu_global();

    input pixel("pixel", {r, cc}, p_float32);
    input tap("tap", {t}, p_float32);
    pixel.store_in(&image_gpu);
    tap.store_in(&taps_gpu);

    computation out("out", {r, c},
                    pixel(r, c) * tap(0) + pixel(r, c + 1) * tap(1) + pixel(r, c + 2) * tap(2) +
                    pixel(r, c + 3) * tap(3) + pixel(r, c + 4) * tap(4));
    out.store_in(&filtered_gpu);
    out.gpu_tile(r, c, 8, 32, rb, cb, rt, ct);

    tiramisu::codegen({&image, &taps, &filtered}, "build/taps_in_constant_memory.o", true);
    return 0;
}
