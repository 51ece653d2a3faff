// NO_CPU_VARIANT (thread loops run serially on the CPU back-end: the element another thread stages does not exist yet)
// out(b, t) = in(b, 63 - t): every workgroup stages its 64 elements in an LDS buffer declared by hand and each
// thread reads the element that the thread at the other end wrote.  `reverse_in_blocks` has the tiramisu::sync
// between the two statements; the generator writes `reverse_in_blocks_unsynced`, the same program without it, only
// when it is run with the argument `unsynced` -- the back-end's race check of shared memory (back-end option
// hip_check_shared_memory) must accept the first and stop code generation of the second.
// sums_over_rounds(b, t) = sum over s < 5 of (in(b, 63 - t) + s) stages the 64 elements again in every round of a serial
// loop inside the kernel: a barrier after the staging and one at the end of the round (the next round overwrites
// what the other thread may still be reading).  `sums_over_rounds_one_sync` (argument `one_sync`) leaves the second
// one out, which the check must find as a read of one round against the write of the next.
#include <cstring>
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

static void reverse_in_blocks(const std::string &name, bool with_sync)
{
    const int N = 4096, T = 64;
    tiramisu::init(name);
    var b("b", 0, N / T), t("t", 0, T);
    input in("in", {b, t}, p_float32);
    in.get_buffer()->tag_gpu_global();
    buffer tile("tile", {T}, p_float32, a_temporary);
    tile.tag_gpu_shared();
    computation tile_decl("tile_decl", {b, t}, allocate(tile));
    computation stage("stage", {b, t}, in(b, t));
    stage.store_in(&tile, {t});
    computation barrier("barrier", {b, t}, tiramisu::sync());
    computation out("out", {b, t}, stage(b, T - 1 - t));
    out.get_buffer()->tag_gpu_global();

    std::vector<computation *> all = {&tile_decl, &stage, &out};
    if (with_sync) all.push_back(&barrier);
    for (computation *c : all) c->tag_gpu_level(b, t);
    if (with_sync) tile_decl.then(stage, t).then(barrier, t).then(out, t);
    else tile_decl.then(stage, t).then(out, t);
    tiramisu::codegen({in.get_buffer(), out.get_buffer()}, "build/" + name + ".o", true);
}

static void sums_over_rounds(const std::string &name, bool closing_sync)
{
    const int N = 4096, T = 64, S = 5;
    tiramisu::init(name);
    var b("b", 0, N / T), t("t", 0, T), s("s", 0, S);
    input in("in", {b, t}, p_float32);
    in.get_buffer()->tag_gpu_global();
    buffer tile("tile", {T}, p_float32, a_temporary);
    tile.tag_gpu_shared();
    computation tile_decl("tile_decl", {b, t}, allocate(tile));
    computation sum_init("sum_init", {b, t}, expr((float)0));
    sum_init.get_buffer()->tag_gpu_global();
    computation stage("stage", {b, t, s}, in(b, t) + cast(p_float32, s));
    stage.store_in(&tile, {t});
    computation staged("staged", {b, t, s}, tiramisu::sync());
    computation sum("sum", {b, t, s}, p_float32);
    sum.store_in(sum_init.get_buffer(), {b, t});
    sum.set_expression(sum(b, t, s - 1) + stage(b, T - 1 - t, s));
    computation consumed("consumed", {b, t, s}, tiramisu::sync());

    std::vector<computation *> all = {&tile_decl, &sum_init, &stage, &staged, &sum};
    if (closing_sync) all.push_back(&consumed);
    for (computation *c : all) c->tag_gpu_level(b, t);
    tile_decl.then(sum_init, t).then(stage, t).then(staged, s).then(sum, s);
    if (closing_sync) sum.then(consumed, s);
    tiramisu::codegen({in.get_buffer(), sum_init.get_buffer()}, "build/" + name + ".o", true);
}

int main(int argc, char **argv)
{
    tiramisu::backend_options_from_command_line(argc, argv);
    bool unsynced = false, one_sync = false;
    for (int i = 1; i < argc; i++) {
        if (!std::strcmp(argv[i], "unsynced")) unsynced = true;
        if (!std::strcmp(argv[i], "one_sync")) one_sync = true;
    }
    reverse_in_blocks("reverse_in_blocks", true);
    sums_over_rounds("sums_over_rounds", true);
    if (unsynced) reverse_in_blocks("reverse_in_blocks_unsynced", false);
    if (one_sync) sums_over_rounds("sums_over_rounds_one_sync", false);
    return 0;
}
