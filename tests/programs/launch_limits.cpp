// NO_CPU_VARIANT (the limits are those of a GPU workgroup)
// What a workgroup can hold, checked when the code is generated (the device compiler accepts more, the launch would
// fail): at most 1024 threads, at most 160 KiB of shared memory.
//  * at_the_limits: 32 x 32 threads, and a shared buffer of 40 x 1024 floats = 163840 bytes that every workgroup fills
//    and reads back reversed: out(b, r, t) = in(b, 39 - r, 1023 - t) -- generated always, and run by the tests;
//  * with the argument `threads` the generator also writes too_many_threads (64 x 64 threads), with `lds`
//    too_much_shared_memory (one float more): code generation must stop at either, naming the kernel and the figure.
#include <cstring>
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

static void reversed_through_lds(const std::string &name, int rows, int extra_floats)
{
    const int NB = 6, T = 1024;
    tiramisu::init(name);
    var b("b", 0, NB), r("r", 0, rows), y("y", 0, 32), x("x", 0, 32);
    input in("in", {b, r, y, x}, p_float32);
    in.get_buffer()->tag_gpu_global();
    buffer tile("tile", {rows * T + extra_floats}, p_float32, a_temporary);
    tile.tag_gpu_shared();
    computation tile_decl("tile_decl", {b, y, x}, allocate(tile));
    computation stage("stage", {b, y, x, r}, in(b, r, y, x));
    stage.store_in(&tile, {r * T + y * 32 + x});
    computation staged("staged", {b, y, x}, tiramisu::sync());
    computation out("out", {b, y, x, r}, stage(b, 31 - y, 31 - x, rows - 1 - r));
    out.get_buffer()->tag_gpu_global();
    for (computation *c : {&tile_decl, &stage, &staged, &out}) {
        c->tag_gpu_block_level(0);
        c->tag_gpu_thread_level(1, 2);
    }
    tile_decl.then(stage, x).then(staged, x).then(out, x);
    tiramisu::codegen({in.get_buffer(), out.get_buffer()}, "build/" + name + ".o", true);
}

static void too_many_threads()
{
    tiramisu::init("too_many_threads");
    var i("i", 0, 256), j("j", 0, 256);
    computation c("c", {i, j}, expr(1) + i);
    c.get_buffer()->tag_gpu_global();
    c.gpu_tile(i, j, 64, 64);
    tiramisu::codegen({c.get_buffer()}, "build/too_many_threads.o", true);
}

int main(int argc, char **argv)
{
    tiramisu::backend_options_from_command_line(argc, argv);
    reversed_through_lds("at_the_limits", 40, 0);
    for (int i = 1; i < argc; i++) {
        if (!std::strcmp(argv[i], "threads")) too_many_threads();
        if (!std::strcmp(argv[i], "lds")) reversed_through_lds("too_much_shared_memory", 40, 1);
    }
    return 0;
}
