// A host time loop that, in every iteration, allocates a GPU buffer, uploads one time slice,
// overwrites it in a kernel mapped with tag_gpu_level, downloads it and frees the buffer; two
// such phases follow each other.  Same features as the reference's tests/test_197.cpp
// (allocate_at / deallocate_at inside a host loop, int32 data, kernels under a host loop).
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

int main()
{
    const int STEPS = 3, PX = 24, QX = 40;
    tiramisu::init("alloc_in_time_loop");

    var t("t", 0, STEPS);
    var p0("p0", 0, PX), p1("p1", 0, PX), q0("q0", 0, QX), q1("q1", 0, QX);

    input P("P", {t, p0, p1}, p_int32);
    input Q("Q", {t, q0, q1}, p_int32);

    buffer dev_P("dev_P", {STEPS, PX, PX}, p_int32, a_temporary);
    buffer dev_Q("dev_Q", {STEPS, QX, QX}, p_int32, a_temporary);
    dev_P.tag_gpu_global();
    dev_Q.tag_gpu_global();

    computation fill_P("fill_P", {t, p0, p1}, expr(7) + p0 * 100 + p1 + t);
    fill_P.store_in(&dev_P, {t, p0, p1});
    fill_P.tag_gpu_level(p0, p1);
    computation fill_Q("fill_Q", {t, q0, q1}, expr(-3) + q0 - q1 * 2 + t);
    fill_Q.store_in(&dev_Q, {t, q0, q1});
    fill_Q.tag_gpu_level(q0, q1);

    computation up_P({t}, memcpy(*P.get_buffer(), dev_P));
    computation up_Q({t}, memcpy(*Q.get_buffer(), dev_Q));
    computation down_P({t}, memcpy(dev_P, *P.get_buffer()));
    computation down_Q({t}, memcpy(dev_Q, *Q.get_buffer()));

    computation *alloc_P = dev_P.allocate_at(up_P, t);
    computation *free_P = dev_P.deallocate_at(down_P, t);
    computation *alloc_Q = dev_Q.allocate_at(up_Q, t);
    computation *free_Q = dev_Q.deallocate_at(down_Q, t);

    alloc_P->then(up_P, t)
            .then(fill_P, t)
            .then(down_P, t)
            .then(*free_P, t)
            .then(*alloc_Q, computation::root)
            .then(up_Q, t)
            .then(fill_Q, t)
            .then(down_Q, t)
            .then(*free_Q, t);

    tiramisu::codegen({P.get_buffer(), Q.get_buffer()}, "build/alloc_in_time_loop.o", true);
    return 0;
}
