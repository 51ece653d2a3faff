// Out-of-place transpose with both loops mapped to the GPU.  Same features as the reference's
// tests/test_168.cpp (a computation that reads an input at swapped indices, gpu_tile).
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

int main()
{
    const int R = 144, S = 80;
    tiramisu::init("transpose_gpu_tile");

    var r("r", 0, R), s("s", 0, S);
    var rb("rb"), rt("rt"), sb("sb"), st("st");

    buffer host_in("host_in", {R, S}, p_float32, a_input);
    buffer host_out("host_out", {S, R}, p_float32, a_output);

    input in({r, s}, p_float32);
    computation out({s, r}, in(r, s));
    in.get_buffer()->tag_gpu_global();
    out.get_buffer()->tag_gpu_global();

    computation upload({}, memcpy(host_in, *in.get_buffer()));
    computation download({}, memcpy(*out.get_buffer(), host_out));

    out.gpu_tile(s, r, 16, 16, sb, rb, st, rt);
    upload.then(out, computation::root).then(download, computation::root);

    tiramisu::codegen({&host_in, &host_out}, "build/transpose_gpu_tile.o", true);
    return 0;
}
