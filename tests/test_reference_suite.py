"""The reference's own test-suite -- generator programs and wrapper programs, both unchanged -- through
this front-end and the CPU emitter of the oracle: every wrapper fills its inputs, calls the generated
function and compares the result with the expectation written by the reference's authors.  This is the
widest check of the front-end (schedule algebra, ordering, access relations, buffer mapping, expression
semantics such as uint8 wrap-around, lerp and clamped accesses) that the reference tree itself holds;
tests/reference_programs/build_reference_programs.py lists the tests and says why the others are absent.
The programs are built beforehand (where the reference tree is present); here they are only run."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "reference_programs"))
import build_reference_programs as brp  # noqa: E402


@pytest.mark.parametrize("n", brp.SUITE + brp.SUITE_TUTORIALS)
def test_reference_test_passes(n):
    program = brp.suite_program(n)
    assert os.path.exists(program), "not built: run tests/reference_programs/build_reference_programs.py where the reference tree is"
    r = subprocess.run([program], cwd=os.path.dirname(program), stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert r.returncode == 0, r.stdout[-2000:]
    assert "failed" not in r.stdout.lower(), r.stdout[-2000:]
    assert "succeeded" in r.stdout or n in brp.SUITE_SILENT, r.stdout[-2000:]
