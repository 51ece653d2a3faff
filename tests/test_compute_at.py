"""compute_at with a redundant duplicate, and storage_fold (tests/programs/compute_at.cpp, CPU emitter): a two-stage
blur, bx(y, x) = in(y, x) + in(y, x+1) + in(y, x+2), by(y, x) = bx(y, x) + bx(y+1, x) + bx(y+2, x), against numpy."""
import os

import numpy as np

from oracle import build as oracle_build
from tiramisu_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAMS = os.path.join(ROOT, "tests", "programs")
H, W = 20, 24


def program(name):
    return runtime.Program(oracle_build.cpu_program_library(PROGRAMS, name), name, needs_gpu_runtime=False)


def blur_inputs(seed):
    image = np.random.RandomState(seed).randint(-50, 50, (H + 2, W + 2)).astype(np.int32)
    bx = image[:, :W] + image[:, 1:W + 1] + image[:, 2:W + 2]
    by = bx[:H] + bx[1:H + 1] + bx[2:H + 2]
    return image, bx, by


def generated_text(name):
    return open(os.path.join(PROGRAMS, "build", name + "_cpu.o.cpu.cpp")).read()


def test_rows_computed_ahead_of_their_reader():
    image, bx, by = blur_inputs(1)
    out_bx, out_by = np.full((H + 2, W), -1, np.int32), np.full((H, W), -1, np.int32)
    program("compute_at_row")(image, out_bx, out_by)
    assert np.array_equal(out_by, by) and np.array_equal(out_bx, bx)
    # one loop nest: the duplicate's row loop starts one iteration before the consumer's
    text = generated_text("compute_at_row")
    assert text.count("for (int32_t c1") == 1 and "c1 = (-1)" in text


def test_halo_rows_of_a_tile():
    image, bx, by = blur_inputs(2)
    out_bx, out_by = np.full((H + 2, W), -1, np.int32), np.full((H, W), -1, np.int32)
    program("compute_at_tile")(image, out_bx, out_by)
    assert np.array_equal(out_by, by) and np.array_equal(out_bx, bx)


def test_nothing_missing_is_ordering_only():
    image = np.random.RandomState(3).randint(-50, 50, (H, W)).astype(np.int32)
    a, c = np.zeros((H, W), np.int32), np.zeros((H, W), np.int32)
    program("compute_at_same")(image, a, c)
    assert np.array_equal(a, 2 * image) and np.array_equal(c, 2 * image + 1)
    text = generated_text("compute_at_same")
    assert "_dup_" not in text and text.count("for (int32_t c3") == 1          # fused down to the innermost loop


def test_storage_fold_keeps_four_rows():
    image, bx, by = blur_inputs(4)
    rows, out_by = np.full((4, W), -1, np.int32), np.full((H, W), -1, np.int32)
    program("storage_fold_rows")(image, rows, out_by)
    assert np.array_equal(out_by, by)
    # what is left in the folded buffer: the last rows written, each at its row number modulo 4
    for r in range(H + 2 - 4, H + 2):
        assert np.array_equal(rows[r % 4], bx[r])
