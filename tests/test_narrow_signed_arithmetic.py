"""Signed 8- and 16-bit products followed by /, % and >> (tests/programs/narrow_signed_arithmetic.cpp).  A Tiramisu
expression keeps its type, so the product wraps before the next operation (the reference's CPU back-end hands Halide
typed expressions, tiramisu_codegen_halide.cpp:1560-1580; its CUDA printer leaves the promotion to C,
tiramisu_codegen_cuda.cpp:1160-1167).  The expectation is numpy's wrapping arithmetic with C's division (towards
zero); the int8 case covers all 65536 pairs of values."""
import os

import numpy as np
import pytest

from oracle import build as oracle_build
from tiramisu_amd import runtime

CASES = {"narrow_products_int8": (np.int8, 1, 1), "narrow_products_int16": (np.int16, 211, 173)}


def inputs_and_expected(dtype, sa, sb):
    i, j = np.meshgrid(np.arange(256) - 128, np.arange(256) - 128, indexing="ij")
    a, b = (i * sa).astype(dtype), (j * sb).astype(dtype)

    def c_div(x, d):
        x = x.astype(np.int64)
        return (np.sign(x) * (np.abs(x) // d))

    prod = (a.astype(np.int64) * b.astype(np.int64)).astype(dtype)
    square = (a.astype(np.int64) * a.astype(np.int64)).astype(dtype)
    half = c_div(prod, 2).astype(dtype)
    rem = (prod.astype(np.int64) - 3 * c_div(prod, 3)).astype(dtype)
    shifted = (prod >> 1).astype(dtype)
    return a, b, [half, rem, shifted, prod, c_div(square, 2).astype(dtype)]


@pytest.mark.parametrize("name", sorted(CASES))
def test_products_pass_through_the_opaque_helper_on_the_device(programs_dir, name):
    text = open(os.path.join(programs_dir, "build", name + ".o.hip")).read()
    assert 'asm("" : "+v"(w))' in text
    ctype = "int8_t" if name.endswith("int8") else "int16_t"
    assert "t_opaque(((%s)(" % ctype in text


@pytest.mark.parametrize("name", sorted(CASES))
def test_cpu_emitter_wraps_the_product_first(programs_dir, name):
    a, b, expected = inputs_and_expected(*CASES[name])
    outs = [np.full(a.shape, 99, a.dtype) for _ in expected]
    runtime.Program(oracle_build.cpu_program_library(programs_dir, name), name, needs_gpu_runtime=False)(a, b, *outs)
    for got, want, what in zip(outs, expected, ("half", "rem", "shifted", "prod", "square_half")):
        assert np.array_equal(got, want), what


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(CASES))
def test_gpu_wraps_the_product_first(programs_dir, name):
    from gpu_util import DeviceArray
    a, b, expected = inputs_and_expected(*CASES[name])
    dev = [DeviceArray(a), DeviceArray(b)] + [DeviceArray(np.full(a.shape, 99, a.dtype)) for _ in expected]
    print(name, flush=True)
    runtime.load(programs_dir, name)(*[d.buffer() for d in dev])
    got = [d.download() for d in dev[2:]]
    for d in dev:
        d.free()
    for g, want, what in zip(got, expected, ("half", "rem", "shifted", "prod", "square_half")):
        assert np.array_equal(g, want), what + ": %d of 65536 differ" % int(np.sum(g != want))
