"""separate / separateAndSplit / separate_at / duplicate (tests/programs/separation.cpp, CPU emitter): every function
computes out(i, j) = 100 i + j over its domain; the generator reports which iterations each piece executes."""
import json
import os

import numpy as np
import pytest

from oracle import build as oracle_build
from tiramisu_amd import runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROGRAMS = os.path.join(ROOT, "tests", "programs")


def run(name, rows, cols):
    out = np.full((rows, cols), -1, np.int32)
    runtime.Program(oracle_build.cpu_program_library(PROGRAMS, name), name, needs_gpu_runtime=False)(out)
    return out


def expected(rows, cols, first_col=0):
    e = np.full((rows, cols), -1, np.int32)
    i, j = np.meshgrid(np.arange(rows), np.arange(first_col, cols), indexing="ij")
    e[:, first_col:] = 100 * i + j
    return e


def pieces(name):
    report = json.load(open(os.path.join(PROGRAMS, "build", "separation.json")))
    return [(p["name"], p["levels"], p["first"], p["last"]) for p in report[name]]


def test_full_part_and_remainder():
    # 14 = 3 x 4 + 2: the split part holds the whole groups, the remainder is a definition of its own, not split
    assert pieces("sep_split") == [("out", 3, 0, 11), ("_out_update_1", 2, 12, 13)]
    assert np.array_equal(run("sep_split", 6, 14), expected(6, 14))


def test_groups_are_counted_from_the_lower_bound():
    # j in [3, 17): 14 iterations again, full part [3, 15)
    assert pieces("sep_lower") == [("out", 3, 3, 14), ("_out_update_1", 2, 15, 16)]
    assert np.array_equal(run("sep_lower", 6, 17), expected(6, 17, first_col=3))


def test_nothing_to_separate():
    assert pieces("sep_exact") == [("out", 3, 0, 15)]
    assert np.array_equal(run("sep_exact", 6, 16), expected(6, 16))
    # a loop of 3 iterations is not split by 4 at all
    assert pieces("sep_short") == [("out", 2, 0, 2)]
    assert np.array_equal(run("sep_short", 6, 3), expected(6, 3))


def test_separate_on_the_outer_loop_and_schedule_the_piece():
    report = json.load(open(os.path.join(PROGRAMS, "build", "separation.json")))["sep_outer"]
    assert [(p["name"], p["first_row"], p["last_row"]) for p in report] == [("out", 0, 3), ("_out_update_1", 4, 5)]
    assert np.array_equal(run("sep_outer", 6, 14), expected(6, 14))


def test_separate_at_points():
    assert pieces("sep_at") == [("out", 2, 0, 3), ("_out_update_1", 2, 4, 8), ("_out_update_2", 2, 9, 13)]
    assert np.array_equal(run("sep_at", 6, 14), expected(6, 14))


def test_duplicate_over_a_part_of_the_domain():
    assert pieces("sep_duplicate") == [("out", 2, 0, 13), ("_out_dup_1", 2, 5, 7)]
    e = expected(6, 14)
    e[2:4, 5:8] += 1000
    assert np.array_equal(run("sep_duplicate", 6, 14), e)
