// Programs that record the order in which a schedule visits its iteration domain: a "stamp"
// computation copies a one-element clock into stamp[i][j] and a "tick" computation, fused with
// it at the innermost loop, advances the clock.  The tests compare the stamps with a
// brute-force enumeration of the schedule's definition (split: tiramisu_core.cpp:6389-6392,
// tile: :2705-2723, interchange: :3119-3181, after/then: :2162-2179 of the reference).
// CPU_ONLY_PROGRAM: compiled only for the CPU back-end restatement: visit order is a property of the shared
// front-end, and a serial execution is what makes it observable.
#include <tiramisu/tiramisu.h>

using namespace tiramisu;

static const int P = 10, Q = 14;

struct recorder {
    var i, j;
    buffer clock_buf, stamp_buf;
    input clock;
    computation stamp, tick;
    recorder(const std::string &fn)
        : i("i", 0, P), j("j", 0, Q), clock_buf("clock_buf", {1}, p_int32, a_output),
          stamp_buf("stamp_buf", {P, Q}, p_int32, a_output), clock("clock", {i, j}, p_int32),
          stamp("stamp", {i, j}, clock(i, j)), tick("tick", {i, j}, clock(i, j) + 1)
    {
        clock.store_in(&clock_buf, {0});
        tick.store_in(&clock_buf, {0});
        stamp.store_in(&stamp_buf, {i, j});
    }
    void finish(const std::string &fn, var innermost) {
        stamp.then(tick, innermost);
        tiramisu::codegen({&clock_buf, &stamp_buf}, "build/" + fn + "_cpu.o", false);
    }
};

int main()
{
    {   // identity
        tiramisu::init("order_identity");
        recorder r("order_identity");
        r.finish("order_identity", r.j);
    }
    {   // split j by 4
        tiramisu::init("order_split");
        recorder r("order_split");
        var jo("jo"), ji("ji");
        r.stamp.split(r.j, 4, jo, ji);
        r.tick.split(r.j, 4, jo, ji);
        r.finish("order_split", ji);
    }
    {   // tile 3x5 (partial tiles on both sides)
        tiramisu::init("order_tile");
        recorder r("order_tile");
        var io("io"), jo("jo"), ii("ii"), ji("ji");
        r.stamp.tile(r.i, r.j, 3, 5, io, jo, ii, ji);
        r.tick.tile(r.i, r.j, 3, 5, io, jo, ii, ji);
        r.finish("order_tile", ji);
    }
    {   // interchange
        tiramisu::init("order_interchange");
        recorder r("order_interchange");
        r.stamp.interchange(r.i, r.j);
        r.tick.interchange(r.i, r.j);
        r.finish("order_interchange", r.i);
    }
    {   // skew j by 2*i, then the loops are still visited in lexicographic (i, j') order
        tiramisu::init("order_skew_shift");
        recorder r("order_skew_shift");
        r.stamp.skew(r.i, r.j, 2);
        r.tick.skew(r.i, r.j, 2);
        r.stamp.shift(r.j, 3);
        r.tick.shift(r.j, 3);
        r.finish("order_skew_shift", r.j);
    }
    {   // two statements ordered at the outer loop only: all stamps of a row, then all ticks
        tiramisu::init("order_fuse_outer");
        recorder r("order_fuse_outer");
        r.finish("order_fuse_outer", r.i);
    }
    {   // vectorize / unroll / parallelize tags must not change what is computed
        tiramisu::init("order_tags");
        recorder r("order_tags");
        var jo("jo"), ji("ji");
        r.stamp.unroll(r.j, 4, jo, ji);
        r.tick.unroll(r.j, 4, jo, ji);
        r.finish("order_tags", ji);
    }
    return 0;
}
