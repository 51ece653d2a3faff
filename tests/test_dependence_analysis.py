"""Dependence analysis and the legality checks built on it (tiramisu_amd/csrc/dependences.cpp; the calls of the
reference's core.h:139-181 and :1236-1330).  tests/programs/dependence_checks.cpp asks them about loops whose
answers can be read off the code -- a wavefront recurrence in place with distances (1,0) and (0,1), the same with
the inner loop reversed, an out-of-place stencil, a producer and a consumer fused into one loop -- and about loops
mapped to GPU threads; its answers are compared here.  The reference's own tests of these calls (tests/test_179 -
test_195, test_198, test_199) run in test_reference_suite.py."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BUILD = os.path.join(ROOT, "tests", "programs", "build")


@pytest.fixture(scope="module")
def answers():
    path = os.path.join(BUILD, "dependence_checks.txt")
    assert os.path.exists(path), "run __graft_entry__.build() first"
    return open(path).read()


def answer(text, what):
    lines = [line for line in text.splitlines() if line.startswith(what + "=")]
    assert len(lines) == 1, what
    return lines[0].split("=", 1)[1]


@pytest.mark.parametrize("what,expected", [
    # S(i,j) = S(i-1,j) + S(i,j-1): legal as written, both loops carry a dependence
    ("wavefront.as_written.legal", "yes"),
    ("wavefront.as_written.i_parallel", "no"),
    ("wavefront.as_written.j_parallel", "no"),
    ("wavefront.as_written.j_unrollable", "yes"),
    ("wavefront.interchanged.legal", "yes"),            # (0,1) and (1,0) stay positive
    # i1 = i + j, j1 = j: distances (1,0), (1,1): the outer loop carries both, the inner one is free; its bounds
    # are now a max and a min of the outer iterator, so it cannot be unrolled (or vectorized) as it stands
    ("wavefront.skewed.legal", "yes"),
    ("wavefront.skewed.outer_parallel", "no"),
    ("wavefront.skewed.inner_parallel", "yes"),
    ("wavefront.skewed.inner_unrollable", "no"),
    ("wavefront.skewed.inner_vectorizable", "no"),
    ("reversed.legal", "no"),                           # (0,1) becomes (0,-1)
    ("out_of_place.tiled.legal", "yes"),
    ("out_of_place.tiled.i0_parallel", "yes"),
    ("out_of_place.tiled.j1_parallel", "yes"),
    # Q(i) = P(i+2): one loop nest after the other is fine, fused Q reads what P has not written yet,
    # delayed by two iterations it reads it right after P wrote it
    ("fusion.one_after_the_other.legal", "yes"),
    ("fusion.fused.legal", "no"),
    ("fusion.fused.P_to_Q_legal", "no"),
    ("fusion.shifts", "1 i:2"),
    ("fusion.shifted.legal", "yes"),
    ("mapped.scale.findings", "0"),
    # the schedule of the reference's tests 133-140: sequentially fine, but the loop they tag parallel carries (1,1)
    ("test_133.order_legal", "yes"),
    ("test_133.ni_parallel", "no"),
    ("test_133.nj_parallel", "no"),
    # skewings from the distances.  (1,0),(0,1): the outer loop carries both when a > 0 and b > 0; no skewing
    # leaves the outer loop free, none keeps a dependence inside it.  (1,1) alone: i - j is constant along it
    ("skewing.wavefront.outer_parallel", "0"),
    ("skewing.wavefront.inner_parallel", "2 (1,1) (1,2)"),
    ("skewing.wavefront.locality", "0"),
    ("skewing.wavefront.positive.inner_parallel", "1 (1,1,0,1)"),
    ("skewing.diagonal.outer_parallel", "1 (1,-1)"),
    ("skewing.diagonal.skewed.legal", "yes"),
    ("skewing.diagonal.skewed.outer_parallel", "yes"),
    ("skewing.out_of_place.total", "0"),
])
def test_answer(answers, what, expected):
    assert answer(answers, what) == expected


def test_dataflow_of_the_wavefront(answers):
    """Every flow dependence has a source and a sink whose coordinates differ by one in exactly one loop; nothing is
    overwritten; row 0 and column 0 are read from outside; every cell written is live at the end."""
    part = answers.split("wavefront.dependences:\n")[1].split("wavefront.interchanged")[0]
    lines = dict(line.split(": ", 1) for line in part.strip().splitlines())
    assert "t1' = 1 + t0 + t1 - t0'" in lines["read_after_write"] and "t0 <= t0'" in lines["read_after_write"] and "t0' <= 1 + t0" in lines["read_after_write"]
    assert lines["write_after_read"].strip() == "{  }" and lines["write_after_write"].strip() == "{  }"
    assert "[0, t1]" in lines["live_in"] and "[t0, 0]" in lines["live_in"]
    assert "S[i, j] -> _A_b0[i, j]" in lines["live_out"]
    out = answers.split("out_of_place.dependences:\n")[1]
    assert out.splitlines()[0].strip() == "read_after_write: {  }"


def test_loops_mapped_to_threads(answers):
    """A scan along a thread loop is a race; a sum along one is reported as a reduction (the back-end lowers it to a
    wavefront reduction); independent points are not reported."""
    assert "mapped.scan_rows: S: loop j (level 1, mapped to threadIdx) carries a dependence through global memory" in answers
    assert "mapped.row_sums: s: loop j (level 1, mapped to threadIdx) carries a reduction through global memory" in answers
    # an index read from a table may name any element: both loops of the permutation in place are refused
    assert "mapped.gather: G: loop k0 (level 0, mapped to blockIdx) carries a dependence" in answers
    assert "mapped.gather: G: loop k1 (level 1, mapped to threadIdx) carries a dependence" in answers
    assert "mapped.scan_rows: S: loop i" not in answers and "mapped.row_sums: s: loop i" not in answers


def test_codegen_refuses_a_race_when_asked_to_check(tmp_path):
    gen = os.path.join(BUILD, "gen_dependence_checks")
    assert os.path.exists(gen), "run __graft_entry__.build() first"
    os.makedirs(tmp_path / "build")
    env = dict(os.environ, TIRAMISU_HIP_CHECK_MAPPED_LOOPS="1")
    r = subprocess.run([gen, "refuse"], cwd=tmp_path, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert r.returncode != 0
    assert "S: loop j (level 1, mapped to threadIdx) carries a dependence" in r.stdout
    assert not os.path.exists(tmp_path / "build" / "scan_rows_refused.o")


def test_the_check_of_mapped_loops_has_a_time_limit(tmp_path):
    """The analysis is one isl dataflow computation over the whole function and has no natural bound; it runs in a child
    process under hip_check_time_limit seconds (default 600).  With a limit of one second the LSTM program's check is
    stopped, says so, and code generation goes on (device and host compilers stubbed out here)."""
    gen = os.path.join(os.path.dirname(BUILD), "..", "..", "tiramisu_amd", "programs", "build", "gen_lstm")
    gen = os.path.abspath(gen)
    assert os.path.exists(gen), "run __graft_entry__.build() first"
    os.makedirs(tmp_path / "build")
    env = dict(os.environ, TIRAMISU_HIP_CHECK_MAPPED_LOOPS="1", TIRAMISU_HIP_CHECK_TIME_LIMIT="1", HIPCC_PATH="/bin/true", TIRAMISU_HOST_CXX="/bin/true")
    r = subprocess.run([gen], cwd=tmp_path, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-2000:]
    assert "the dependence analysis of lstm_4x64x512x100 did not finish within 1 s and was stopped" in r.stdout
    assert os.path.exists(tmp_path / "build" / "lstm_4x64x512x100.o.hip")
