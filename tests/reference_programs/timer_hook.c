/* get_time(): the external timer that the reference's GPU benchmark programs call from generated
 * host code (expr(o_call, "get_time", ...) in benchmarks/linear_algebra/blas/level3/sgemm/gpu/
 * generator3.cpp:66-67; their wrappers define it).  Milliseconds since the first call. */
#include <stdint.h>
#include <time.h>

float get_time(int32_t dummy)
{
    static struct timespec t0;
    static int started = 0;
    struct timespec t;
    (void)dummy;
    clock_gettime(CLOCK_MONOTONIC, &t);
    if (!started) { t0 = t; started = 1; }
    return (float)((t.tv_sec - t0.tv_sec) * 1e3 + (t.tv_nsec - t0.tv_nsec) * 1e-6);
}
