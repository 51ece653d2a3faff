"""Time candidates of a Tiramisu program on the GPU: the Python side of evaluation by execution (the
reference's src/auto_scheduler/tiramisu_evaluator.cpp: build the candidate, run it, keep the time).  The
evaluator itself is C++ (tiramisu::auto_scheduler::evaluate_by_execution, include/tiramisu/auto_scheduler/
evaluator.h); what lives here is

  * the wrapper that the C++ evaluator runs:  python -m tiramisu_amd.autotune --time LIBRARY FUNCTION [MANIFEST]
    loads the library, calls the function on seeded integer-valued inputs shaped after the back-end's description
    of its arguments and prints one time in milliseconds per run (--outputs FILE.npz keeps the outputs);
  * build_tuner / run_tuner for the compiled tuners of tiramisu_amd/tuning (square_tiles.cpp drives the C++
    evaluator over the MFMA kernel's square tiles and checks the back-end's tile model);
  * a sweeper for generator programs whose main() passes its arguments to
    tiramisu::backend_options_from_command_line:

        python -m tiramisu_amd.autotune tiramisu_amd/programs/heat2d.cpp heat2d_8192x32 \\
            --option stencil_steps=7,9,11 --option stencil_rows=8,10,11

    builds the generator once, runs it once per combination of option values ("--backend-option name=value"
    arguments: candidates are option sets, nothing goes through the environment), and prints one line per
    candidate, fastest first.  Every candidate's outputs are compared with the first one's: an option must not
    change results (integer-valued inputs, so contraction kernels compare exactly too).
Options: stencil_steps / _rows / _waves / _merge / _xcd / _stream, mfma_tile / _bk / _pad / _depth / _wgk,
no_mfma, no_stencil, hip_serial_host_loops (function::set_backend_option in include/tiramisu/core.h)."""
import argparse
import itertools
import json
import os
import shutil
import subprocess
import sys
import tempfile

import numpy as np

from . import build, runtime


def variants(knobs):
    names = [k.split("=", 1)[0] for k in knobs]
    values = [k.split("=", 1)[1].split(",") for k in knobs]
    for combo in itertools.product(*values):
        yield dict(zip(names, combo))


def generate(gen, directory, options):
    """Run generator `gen` in `directory` with the candidate's options as --backend-option arguments."""
    os.makedirs(os.path.join(directory, "build"), exist_ok=True)
    args = []
    for k, v in options.items():
        args += ["--backend-option", "%s=%s" % (k, v)]
    subprocess.run([gen] + args, cwd=directory, check=True, stdout=subprocess.DEVNULL)


def link(directory, function):
    obj = os.path.join(directory, "build", function + ".o")
    if not os.path.exists(obj):
        obj = os.path.join(directory, "build", "generated_fct_" + function + ".o")
    lib = os.path.join(directory, "build", "lib%s.so" % function)
    subprocess.run(["g++", "-shared", "-o", lib, obj, "-L" + build.PKG, "-ltiramisu_hip_wrappers", "-Wl,-rpath," + build.PKG], check=True)
    return lib


class DeviceBuffer:
    def __init__(self, host):
        self.w = runtime.wrappers()
        self.host = np.ascontiguousarray(host)
        self.ptr = self.w.tiramisu_hip_malloc(max(self.host.nbytes, 16))
        self.upload()

    def upload(self):
        self.w.tiramisu_hip_memcpy_to_device(self.ptr, self.host.ctypes.data, self.host.nbytes)

    def download(self):
        out = np.empty_like(self.host)
        self.w.tiramisu_hip_stream_synchronize(0)
        self.w.tiramisu_hip_memcpy_to_host(out.ctypes.data, self.ptr, out.nbytes)
        return out

    def free(self):
        self.w.tiramisu_hip_free(self.ptr)


def make_arguments(manifest, seed):
    rng = np.random.RandomState(seed)
    args = []
    for a in manifest["arguments"]:
        if not all(isinstance(v, int) for v in a["shape"]):
            raise SystemExit("argument %s has run-time extents %s: the harness needs constant shapes" % (a["name"], a["shape"]))
        dtype = np.dtype(runtime._C_TYPES[a["type"]])
        values = rng.randint(0, 4, a["shape"]) if dtype.kind in "iu" else rng.randint(-2, 3, a["shape"])
        host = values.astype(dtype)
        args.append(DeviceBuffer(host) if a["memory"] == "device" else host)
    return args


class evaluate_by_execution:
    """Evaluation of a candidate by running it on the GPU: the counterpart of the reference's
    tiramisu::auto_scheduler::evaluate_by_execution (include/tiramisu/auto_scheduler/evaluator.h,
    src/auto_scheduler/tiramisu_evaluator.cpp:14-72 -- apply the candidate's optimisations, compile the
    program to an object, turn it into a shared library, run it, return the time).  A candidate here is
    a set of back-end options ({name: value}, handed to the generator as --backend-option arguments, which
    tiramisu::backend_options_from_command_line turns into function::set_backend_option calls) instead of a
    syntax tree of schedule transformations; `evaluate` returns the median
    time of one call in milliseconds (HIP events on the calling stream), `get_measurements` every
    sample, as the reference's method of the same name does (:74-125).

    `prepare` does the part that needs no GPU (run the generator under the candidate's options, which
    calls hipcc, and link the library) and keeps its result in `directory`/<candidate>/ so that it can
    run ahead of time on a machine without a GPU; `evaluate` prepares what is not there yet.  The
    outputs of the last evaluated candidate stay in `last_outputs` (inputs are seeded, integer-valued:
    candidates can be compared bit for bit)."""

    def __init__(self, source, function, directory, repeat=20, seed=1):
        self.source, self.function, self.directory = os.path.abspath(source), function, os.path.abspath(directory)
        self.repeat, self.seed = repeat, seed
        self.last_outputs, self.last_kernels = None, None

    @staticmethod
    def candidate_name(candidate):
        return "_".join("%s-%s" % (k, candidate[k]) for k in sorted(candidate)) or "default"

    def library(self, candidate):
        return os.path.join(self.directory, self.candidate_name(candidate), "build", "lib%s.so" % self.function)

    def prepare(self, candidate, force=False):
        lib = self.library(candidate)
        newest_input = max(os.path.getmtime(self.source), os.path.getmtime(build.compiler_library()))
        if os.path.exists(lib) and os.path.getmtime(lib) >= newest_input and not force:
            return lib
        os.makedirs(self.directory, exist_ok=True)
        gen = os.path.join(self.directory, "generator")
        if force or not os.path.exists(gen) or os.path.getmtime(gen) < newest_input:
            subprocess.run(["g++", "-std=c++17", "-O1", "-I" + build.INCLUDE, "-I" + os.path.dirname(self.source), "-o", gen,
                            self.source, "-L" + build.PKG, "-ltiramisu", "-Wl,-rpath," + build.PKG], check=True)
        directory = os.path.join(self.directory, self.candidate_name(candidate))
        generate(gen, directory, {k: str(v) for k, v in candidate.items()})
        return link(directory, self.function)

    def options_used(self, candidate):
        """The options that code generation found set for this candidate, from the manifest."""
        return {o["name"]: o["value"] for o in runtime.manifest_of(self.library(candidate), self.function).get("options", [])}

    def get_measurements(self, candidate, repeat=None):
        lib = self.prepare(candidate)
        manifest = runtime.manifest_of(lib, self.function)
        program = runtime.Program(lib, self.function)
        args = make_arguments(manifest, self.seed)

        def call():
            program(*[runtime.Buffer.from_device(a.ptr, a.host.shape, a.host.dtype) if isinstance(a, DeviceBuffer) else a for a in args])
        call()
        self.last_outputs = [(a.download() if isinstance(a, DeviceBuffer) else a.copy())
                             for a, m in zip(args, manifest["arguments"]) if m["kind"] == "output"]
        self.last_kernels = [k["how"] for k in manifest["kernels"]]
        repeat = repeat or self.repeat
        for _ in range(max(3, repeat // 2)):
            call()
        times = []
        for _ in range(repeat):
            with runtime.DeviceTimer() as t:
                call()
            times.append(t.ms)
        for a in args:
            if isinstance(a, DeviceBuffer):
                a.free()
        return times

    def evaluate(self, candidate):
        return float(np.median(self.get_measurements(candidate)))


def time_library(library, function, manifest_path=None, repeat=20, seed=1, outputs=None):
    """The wrapper of the C++ evaluator: one time in milliseconds per run on standard output."""
    if runtime.wrappers().tiramisu_hip_device_count() < 1:
        raise SystemExit("no HIP device visible")
    manifest = json.load(open(manifest_path)) if manifest_path else runtime.manifest_of(library, function)
    program = runtime.Program(library, function)
    program.manifest = manifest
    args = make_arguments(manifest, seed)

    def call():
        program(*[runtime.Buffer.from_device(a.ptr, a.host.shape, a.host.dtype) if isinstance(a, DeviceBuffer) else a for a in args])
    call()
    if outputs:
        np.savez(outputs, **{m["name"]: (a.download() if isinstance(a, DeviceBuffer) else a)
                             for a, m in zip(args, manifest["arguments"])},
                 **{"input_" + m["name"]: a.host for a, m in zip(args, manifest["arguments"]) if isinstance(a, DeviceBuffer) and m["kind"] == "input"})
    for _ in range(max(3, repeat // 2)):
        call()
    for _ in range(repeat):
        with runtime.DeviceTimer() as t:
            call()
        print("%.6f" % t.ms, flush=True)
    for a in args:
        if isinstance(a, DeviceBuffer):
            a.free()


TUNING = os.path.join(build.PKG, "tuning")


def build_tuner(name):
    """Compile tiramisu_amd/tuning/<name>.cpp against the compiler library (no GPU needed); returns the executable."""
    src = os.path.join(TUNING, name + ".cpp")
    out = os.path.join(TUNING, "build", name)
    os.makedirs(os.path.dirname(out), exist_ok=True)
    if not os.path.exists(out) or os.path.getmtime(out) < max(os.path.getmtime(src), os.path.getmtime(build.compiler_library())):
        subprocess.run(["g++", "-std=c++17", "-O1", "-I" + build.INCLUDE, "-o", out, src, "-L" + build.PKG, "-ltiramisu",
                        "-Wl,-rpath," + build.PKG], check=True)
    return out


def run_tuner(name, scratch, *args):
    """Run a compiled tuner on the GPU machine; returns its JSON lines."""
    os.makedirs(scratch, exist_ok=True)
    env = dict(os.environ)
    env["PYTHONPATH"] = build.ROOT + os.pathsep + env.get("PYTHONPATH", "")
    out = subprocess.run([build_tuner(name), scratch] + [str(a) for a in args], check=True, stdout=subprocess.PIPE, text=True, env=env, cwd=build.ROOT).stdout
    return [json.loads(l) for l in out.splitlines() if l.startswith("{")]


def main(argv=None):
    argv = sys.argv[1:] if argv is None else argv
    if argv and argv[0] == "--time":
        ap = argparse.ArgumentParser()
        ap.add_argument("--time", action="store_true")
        ap.add_argument("library")
        ap.add_argument("function")
        ap.add_argument("manifest", nargs="?")
        ap.add_argument("--repeat", type=int, default=20)
        ap.add_argument("--outputs")
        a = ap.parse_args(argv)
        return time_library(a.library, a.function, a.manifest, a.repeat, outputs=a.outputs)
    if argv and argv[0] == "--tuner":
        for line in run_tuner(argv[1], argv[2], *argv[3:]):
            print(json.dumps(line))
        return
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("source")
    ap.add_argument("function")
    ap.add_argument("--option", "--knob", dest="knob", action="append", default=[], help="name=v1,v2,...")
    ap.add_argument("--repeat", type=int, default=20)
    ap.add_argument("--keep", help="directory to keep the generated variants in")
    a = ap.parse_args(argv)
    if runtime.wrappers().tiramisu_hip_device_count() < 1:
        raise SystemExit("no HIP device visible")
    scratch = a.keep or tempfile.mkdtemp(prefix="tiramisu_autotune_")
    evaluator = evaluate_by_execution(a.source, a.function, scratch, repeat=a.repeat)
    results, first = [], None
    for candidate in variants(a.knob):
        ms = evaluator.evaluate(candidate)
        same = True
        if first is None:
            first = evaluator.last_outputs
        else:
            same = all(np.array_equal(x, y) for x, y in zip(first, evaluator.last_outputs))
        results.append({"options": candidate, "ms": ms, "same_as_first": same, "kernels": [k.split(",")[0] for k in evaluator.last_kernels]})
    results.sort(key=lambda r: r["ms"])
    for r in results:
        print(json.dumps(r))
    if not a.keep:
        shutil.rmtree(scratch, ignore_errors=True)
    return results


if __name__ == "__main__":
    main()
