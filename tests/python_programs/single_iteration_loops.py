"""Programs whose GPU-tagged loops all have a single iteration, so that isl's AST holds no loop for them (the
reference leaves the case open: "TODO check if degenerate", tiramisu_codegen_cuda.cpp:252): the statements must
still run in a kernel -- of one workgroup -- and not on the host with their GPU buffers.
  single_point_py:    tmp = a + 1, out = tmp * tmp - a on a domain of one point, both tiled 1 x 4 and fused;
  single_point_steps_py: out[t] = a[t] * 2 + t, a host loop over t around a tiled domain of one point (the kernel is
                      launched once per step with t as its parameter).
Run at build time; writes the objects and libraries under build/ next to this file."""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(HERE)), "tiramisu_amd", "python"))

from tiramisu import *  # noqa: E402,F403

I32 = primitive_t.p_int32
os.makedirs(os.path.join(HERE, "build"), exist_ok=True)


def device(name, shape, kind):
    b = buffer(name, [expr(s) for s in shape], I32, kind)
    b.tag_gpu_global()
    return b


init("single_point_py")
i, j = var("i", 0, 1), var("j", 0, 1)
i0, j0, i1, j1 = var("i0"), var("j0"), var("i1"), var("j1")
a, tb, o = device("a", (1, 1), argument_t.a_input), device("tb", (1, 1), argument_t.a_temporary), device("o", (1, 1), argument_t.a_output)
A = input("A", [i, j], I32)
A.store_in(a)
tmp = computation("tmp", [i, j], A[i, j] + 1)
out = computation("out", [i, j], I32)
out.set_expression(tmp[i, j] * tmp[i, j] - A[i, j])
tmp.store_in(tb)
out.store_in(o)
tmp.gpu_tile(i, j, 1, 4, i0, j0, i1, j1)
out.gpu_tile(i, j, 1, 4, i0, j0, i1, j1)
tmp.then(out, j1)
pycodegen([a, o], os.path.join(HERE, "build", "single_point_py.o"), True)

STEPS = 5
init("single_point_steps_py")
t, i, j = var("t", 0, STEPS), var("i", 0, 1), var("j", 0, 1)
i0, j0, i1, j1 = var("i0"), var("j0"), var("i1"), var("j1")
a, o = device("a", (STEPS,), argument_t.a_input), device("o", (STEPS,), argument_t.a_output)
ta = var("ta", 0, STEPS)
A = input("A", [ta], I32)
A.store_in(a)
out = computation("out", [t, i, j], A[t] * 2 + t)
out.store_in(o, [t])
out.gpu_tile(i, j, 2, 2, i0, j0, i1, j1)
pycodegen([a, o], os.path.join(HERE, "build", "single_point_steps_py.o"), True)
