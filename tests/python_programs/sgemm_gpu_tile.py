"""C = alpha * A * B + beta * C in fp32, written with the Python front-end (API of the reference's
python_bindings; program structure of its tutorials/tutorial_04A.py) and scheduled for the GPU:
(i, j) tiled 16x16 onto blocks and threads, one register accumulator per thread.  Run at build
time; writes build/sgemm_py.o and links build/libsgemm_py.so next to this file."""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(HERE)), "tiramisu_amd", "python"))

from tiramisu import *  # noqa: E402,F403

M, N, K = 192, 128, 96

init("sgemm_py")

i, j, k, s = var("i", 0, M), var("j", 0, N), var("k", 0, K), var("s", 0, 2)
ib, jb, it, jt = var("ib"), var("jb"), var("it"), var("jt")

b_scal = buffer("b_scal", [expr(2)], primitive_t.p_float32, argument_t.a_input)
b_A = buffer("b_A", [expr(M), expr(K)], primitive_t.p_float32, argument_t.a_input)
b_B = buffer("b_B", [expr(K), expr(N)], primitive_t.p_float32, argument_t.a_input)
b_C = buffer("b_C", [expr(M), expr(N)], primitive_t.p_float32, argument_t.a_output)
acc_reg = buffer("acc_reg", [expr(1)], primitive_t.p_float32, argument_t.a_temporary)
for b in (b_A, b_B, b_C):
    b.tag_gpu_global()
acc_reg.tag_gpu_register()

scal = input("scal", [s], primitive_t.p_float32)
scal.store_in(b_scal)
alpha = constant("alpha", scal[0])
beta = constant("beta", scal[1])
A = input("A", [i, k], primitive_t.p_float32)
B = input("B", [k, j], primitive_t.p_float32)
A.store_in(b_A)
B.store_in(b_B)

acc_decl = computation("acc_decl", [i, j], allocate(acc_reg))
acc_init = computation("acc_init", [i, j], expr(0.0))
acc = computation("acc", [i, j, k], primitive_t.p_float32)
acc.set_expression(acc[i, j, 0] + A[i, k] * B[k, j])
C = computation("C", [i, j], primitive_t.p_float32)
C.set_expression(acc[i, j, 0] * alpha + C[i, j] * beta)

acc_init.store_in(acc_reg, [expr(0)])
acc.store_in(acc_reg, [expr(0)])
C.store_in(b_C)

for c in (acc_decl, acc_init, acc, C):
    c.gpu_tile(i, j, 16, 16, ib, jb, it, jt)
acc_decl.then(acc_init, jt).then(acc, jt).then(C, jt)

os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
pycodegen([b_scal, b_A, b_B, b_C], os.path.join(HERE, "build", "sgemm_py.o"), True)
