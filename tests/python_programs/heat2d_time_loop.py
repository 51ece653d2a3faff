"""The heat2d time loop (out = 0.2 * (c + n + s + w + e), fixed boundary, ping-pong planes indexed
t % 2) written with the Python front-end; same program text as tiramisu_amd/programs/heat2d.cpp.
Run at build time; writes build/heat2d_py.o and links build/libheat2d_py.so next to this file."""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(HERE)), "tiramisu_amd", "python"))

from tiramisu import *  # noqa: E402,F403

N, STEPS = 130, 5

init("heat2d_py")

t, y, x = var("t", 1, STEPS + 1), var("y", 1, N - 1), var("x", 1, N - 1)
yb, xb, yt, xt = var("yb"), var("xb"), var("yt"), var("xt")

planes = buffer("planes", [expr(2), expr(N), expr(N)], primitive_t.p_float32, argument_t.a_output)
planes.tag_gpu_global()

heat = computation("heat", [t, y, x], primitive_t.p_float32)
heat.set_expression((heat[t - 1, y, x] + heat[t - 1, y - 1, x] + heat[t - 1, y + 1, x] +
                     heat[t - 1, y, x - 1] + heat[t - 1, y, x + 1]) * expr(0.2))
heat.store_in(planes, [t % 2, y, x])
heat.gpu_tile(y, x, 16, 16, yb, xb, yt, xt)

os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
pycodegen([planes], os.path.join(HERE, "build", "heat2d_py.o"), True)
