#!/usr/bin/env python3
"""Benchmark of the Tiramisu HIP back-end on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|heat2d|sgemm1024|sgemm4096|...]

Prints ONE JSON line.  The headline is benchmark configuration 2 (heat2d 8192x8192, 32 time steps,
the configuration the HBM-roofline target is quoted on).  A "step" is one call of the compiled
Tiramisu function (32 stencil time steps) with its buffers already resident in HBM.  The compiled
function fuses up to 12 time steps per launch, so it moves far fewer bytes than the un-fused
program's 8 bytes per cell and time step: `value` is the HBM traffic the function really causes
(hardware counters, per kernel, from profiles/hbm_traffic_by_kernel.md) per second, and
`algorithmic_gbs` -- the un-fused program's bytes per second of this run, the figure that time
tiling raises above the HBM peak -- is kept beside it.  The other configurations that exist as
compiled programs are measured the same way and reported under "workloads".

`roofline` is for the kernel with the largest share of the time, its duration measured here with
HIP events around every launch (the runtime ABI's tiramisu_hip_profile_*) on the stream the
generated code launches on: flops per launch over duration against the MFMA peak for the
contractions; counter-measured HBM bytes per launch over duration against the HBM peak for the
stencil (`frac` <= 1 by construction; `algorithmic_gbs` and `vector_alu_busy` say why a fused
launch sits below the HBM peak).  For the contractions the launch duration is the smaller of that and the
timed call minus the other kernels over the kernel's launches: events between the launches of a dependent
chain (the LSTM's cell kernel) or around a kernel of a few microseconds (sgemm 1024^3) cost a good part of a
launch themselves; the per-event figure stays in `kernel_ms_between_events`.  `traffic` is looked up by the emitter's own description of the
kernel, so a kernel the table does not know reports null instead of a stale figure.
`cpu_baseline` times the CPU-generated code of the same Tiramisu program (the oracle's CPU
back-end restatement: parallelize + vectorize schedule, OpenMP) on the host cores of this machine.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import numpy as np  # noqa: E402

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
FP32_MFMA_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix
BF16_MFMA_PEAK_TFLOPS = 2500.0
FP32_VALU_PEAK_TFLOPS = 157.3  # MI355X vector fp32 (256 CUs x 128 lanes x 2 flops x 2.4 GHz): what a kernel without MFMA is priced against
FP32_VALU_PLAIN_TFLOPS = 39.3  # 256 CUs x 64 lanes x 2.4 GHz x 1 flop: separate adds and multiplies, one per lane and clock (no FMA:
                               # the stencil's value must round as the un-fused program's; packed fp32 is not used on this pool)
PROGRAMS = os.path.join(ROOT, "tiramisu_amd", "programs")

TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "hbm_traffic_by_kernel.md")


def traffic_table():
    """{(function, kernel description): {"bytes": HBM bytes per launch, "vector_alu_busy": share or None, "source": hash}}
    from the table of counter measurements in profiles/ (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per dispatch,
    scaled by what the same counters read for a plain copy of known size).  "source" is kernel_source_hash() of
    the function at the time of the measurement."""
    out = {}
    if not os.path.exists(TRAFFIC_TABLE):
        return out
    for line in open(TRAFFIC_TABLE):
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if len(cells) < 7 or not cells[4].replace(".", "", 1).isdigit():
            continue
        busy = cells[5].rstrip("%").strip()
        out[(cells[0].strip("`"), cells[1].strip("`"))] = {
            "bytes": float(cells[4]), "vector_alu_busy": float(busy) / 100.0 if busy.replace(".", "", 1).isdigit() else None,
            "source": cells[6].strip("`")}
    return out


def kernel_source_hash(name):
    """Twelve hex digits over the generated device source of a function and the kernel headers it includes: a
    counter measurement belongs to exactly this text."""
    import hashlib
    import re
    text = open(os.path.join(PROGRAMS, "build", name + ".o.hip")).read()
    # kernel headers are included by file name (the device compiler gets their directory); the hash is taken over
    # the text with the directory spelled "kernels/", as generated code of earlier versions named it by path
    text = re.sub(r'#include "(?:[^"]*/kernels/)?([A-Za-z0-9_]+\.hip\.h)"', r'#include "kernels/\1"', text)
    h = hashlib.sha1(text.encode())
    for inc in sorted(set(re.findall(r'#include "(kernels/[^"]+)"', text))):
        path = os.path.join(ROOT, "tiramisu_amd", "csrc", "kernels", os.path.basename(inc))
        h.update(open(path, "rb").read())
    return h.hexdigest()[:12]


def kernel_descriptions(name):
    """{kernel name: the emitter's description of it} from the manifest written beside the object."""
    with open(os.path.join(PROGRAMS, "build", name + ".o.json")) as f:
        return {k["name"]: k["how"] for k in json.load(f)["kernels"]}


def kernel_traffic(name, kernel):
    """The counter record of a kernel, or None when there is none for this description or the kernel's source
    has changed since it was measured."""
    row = traffic_table().get((name, kernel_descriptions(name).get(kernel, "")))
    if row and row["source"] != kernel_source_hash(name):
        return None
    return row


def device_array(host):
    from gpu_util import DeviceArray
    return DeviceArray(host)


CLOCK_RAMP_SECONDS = 0.25   # a cold GPU raises its clocks over tens of milliseconds of load
EXTRA_WARMUP = {}           # "last": untimed steps the latest time_steps() ran beyond --warmup to cover the ramp


def time_steps(call, steps, warmup):
    """`warmup` untimed steps -- continued, still untimed, until CLOCK_RAMP_SECONDS of load have
    passed, so that short workloads are not timed while the clocks still ramp -- then exactly
    `steps` timed steps between two stream synchronisations."""
    from tiramisu_amd import runtime
    w = runtime.wrappers()
    t_warm = time.perf_counter()
    for _ in range(warmup):
        call()
    w.tiramisu_hip_stream_synchronize(0)
    extra = 0
    while time.perf_counter() - t_warm < CLOCK_RAMP_SECONDS and extra < 100000:
        for _ in range(10):
            call()
        extra += 10
        w.tiramisu_hip_stream_synchronize(0)
    EXTRA_WARMUP["last"] = extra
    t0 = time.perf_counter()
    for _ in range(steps):
        call()
    w.tiramisu_hip_stream_synchronize(0)
    return (time.perf_counter() - t0) * 1e3 / steps


def kernel_profile(call, steps):
    """Average duration per kernel name over `steps` calls, HIP events around every launch."""
    from tiramisu_amd import runtime
    recs = runtime.profile(lambda: [call() for _ in range(steps)])
    by = {}
    for name, ms in recs:
        by.setdefault(name, []).append(ms)
    return {k: (float(np.mean(v)), len(v) // steps) for k, v in by.items()}


def launch_duration(prof, dominant, ms_per_call):
    """(milliseconds per launch of the dominant kernel, how it was obtained).  HIP events around every launch
    include what an event costs between two launches; the timed calls (no events inside) bound the kernel
    from above as well: the call minus the other kernels, over this kernel's launches.  The smaller of the two
    is the one a kernel trace agrees with (a chain of dependent launches, or a kernel of a few microseconds);
    the other kernels' event times carry the same overhead, so the subtraction leans low: the roofline entry
    also carries `frac_between_events`, the fraction on the per-event duration, as the conservative figure."""
    per_event, launches = prof[dominant]
    others = sum(v[0] * v[1] for k, v in prof.items() if k != dominant)
    from_calls = (ms_per_call - others) / launches
    if 0.0 < from_calls < per_event:
        return from_calls, "HIP events around the timed calls, minus the other kernels, over this kernel's launches"
    return per_event, "HIP events around each launch"


def cpu_time(call, min_seconds=3.0, max_runs=5, warm=True):
    if warm:
        call()  # warm-up
    ts = []
    t_all = time.perf_counter()
    while len(ts) < max_runs and (len(ts) < 1 or time.perf_counter() - t_all < min_seconds):
        t0 = time.perf_counter()
        call()
        ts.append(time.perf_counter() - t0)
    return float(np.median(ts)), len(ts)


def cpu_threads():
    return int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))


# ---------------------------------------------------------------- workloads

def stencil_kernels(kernel_source, domain_cells):
    """{kernel name: (time steps fused in one launch, cells advanced per launch, planes read or
    written per launch)}, read from the emitter's description of each kernel in the generated
    kernel source: the kernel for interior tiles advances tiles x tile extent cells, its companion
    the rest of the iteration domain -- or the one launch all of it, when it carries the boundary
    slices behind its interior tiles.  A launch reads one plane and writes one; the launch that
    ends the time loop writes two (the last step and the last but one)."""
    import re
    text = open(kernel_source).read()
    out = {}
    for m in re.finditer(r"// (\w+): stencil: (\d+) time step\(s\) per launch, radius \d+, tile (\d+)x(\d+) in registers, "
                         r".*?, (\d+) interior tiles([^\n]*)", text):
        out[m.group(1)] = (int(m.group(2)), int(m.group(3)) * int(m.group(4)) * int(m.group(5)), 3 if "into both planes" in m.group(6) else 2)
    for m in re.finditer(r"// (\w+): stencil: the \d+ tiles of (\w+)'s launch[^\n]*", text):
        steps, cells, planes = out[m.group(2)]
        if "carried by" in m.group(0):          # one launch advances the whole iteration domain
            out[m.group(2)] = (steps, domain_cells, planes)
        else:
            out[m.group(1)] = (steps, domain_cells - cells, planes)
    return out


def stencil_arithmetic(kernel_source):
    """{kernel name: (floating-point operations of the stencil expression per cell and step, cells that a launch
    stages = computes at every one of its steps, halo and stale cells included)} from the generated kernel source:
    the operators of ST_EXPR, and the tile geometry in the emitter's descriptions (a workgroup stages wavefronts x
    rows x 256 cells; a boundary slice stages its rows + 2 x steps x radius)."""
    import re
    text = open(kernel_source).read()
    out = {}
    for m in re.finditer(r"// (\w+): stencil: (\d+) time step\(s\) per launch, radius (\d+), tile \d+x\d+ in registers, (\d+) wavefronts x (\d+) rows, "
                         r"(\d+) interior tiles[^\n]*\n(?:#define [^\n]*\n)*?#define ST_EXPR ([^\n]*)", text):
        name, steps, radius = m.group(1), int(m.group(2)), int(m.group(3))
        staged = int(m.group(6)) * int(m.group(4)) * int(m.group(5)) * 256
        e = re.search(r"// \w+: stencil: the (\d+) tiles of %s's launch[^\n]*in (\d+) slice\(s\) of (\d+) rows each[^\n]*carried by" % name, text)
        if e:
            staged += int(e.group(1)) * int(e.group(2)) * (int(e.group(3)) + 2 * steps * radius) * 256
        out[name] = (len(re.findall(r" [-+*/] ", m.group(7))), staged)
    return out


def bench_heat2d(steps, warmup, with_cpu):
    from tiramisu_amd import runtime
    from oracle import build as oracle_build
    n, tsteps = 8192, 32
    name = "heat2d_%dx%d" % (n, tsteps)
    rng = np.random.RandomState(2)
    planes = np.zeros((2, n, n), np.float32)
    planes[0, 1:-1, 1:-1] = rng.uniform(0.0, 1.0, (n - 2, n - 2)).astype(np.float32)
    dev = device_array(planes)
    prog = runtime.load(PROGRAMS, name)
    buf = dev.buffer()
    ms = time_steps(lambda: prog(buf), steps, warmup)
    alg_bytes = tsteps * 2.0 * n * n * 4
    prof = kernel_profile(lambda: prog(buf), steps)
    # dominant kernel: the one with the largest total time per call
    dom = max(prof.items(), key=lambda kv: kv[1][0] * kv[1][1])
    # algorithmic bytes of one launch: every cell the kernel advances is read once and written once per step
    described = stencil_kernels(os.path.join(PROGRAMS, "build", name + ".o.hip"), (n - 2) * (n - 2))
    fused_steps, cells, planes_moved = described[dom[0]]
    per_launch_alg = fused_steps * 2.0 * cells * 4
    # a fused launch cannot do with less than one read of the plane and one write of each plane it leaves
    minimum = {k: described[k][2] * n * n * 4.0 for k in prof}
    fused_min = minimum[dom[0]]
    measured = {k: kernel_traffic(name, k) for k in prof}
    t_dom = measured[dom[0]]
    # whole function: counter bytes of every launch; the fused minimum stands in for a kernel the table does not know
    call_bytes = sum((measured[k]["bytes"] if measured[k] else minimum[k]) * v[1] for k, v in prof.items())
    dom_bytes = t_dom["bytes"] if t_dom else None
    hbm_gbs = (dom_bytes if dom_bytes else fused_min) / (dom[1][0] * 1e-3) / 1e9
    # what the launch computes: every cell of the domain at every fused step (useful), and every cell it stages
    # at every step (what the vector ALUs really execute: halo and stale cells included)
    ops, staged_cells = stencil_arithmetic(os.path.join(PROGRAMS, "build", name + ".o.hip"))[dom[0]]
    useful_tflops = cells * fused_steps * ops / (dom[1][0] * 1e-3) / 1e12
    staged_tflops = staged_cells * fused_steps * ops / (dom[1][0] * 1e-3) / 1e12
    dev.free()
    rates = streaming_rates()
    hbm = {"achieved": hbm_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": hbm_gbs / HBM_PEAK_GBS,
           "traffic": dom_bytes, "traffic_basis": "hardware counters of profiles/hbm_traffic_by_kernel.md (same kernel source)" if dom_bytes
                      else "none for this kernel source: the read-once-write-once minimum stands in",
           "fused_minimum_bytes": fused_min, "traffic_over_fused_minimum": dom_bytes / fused_min if dom_bytes else None,
           "streaming_ceiling_gbs": rates["ceiling"], "frac_of_streaming_ceiling": hbm_gbs / rates["ceiling"],
           "algorithmic_gbs": per_launch_alg / (dom[1][0] * 1e-3) / 1e9}
    if fused_steps == 1:
        roofline = dict(hbm, bound="hbm")
        roofline["limiter"] = "hbm: %.0f GB/s against %.0f GB/s for the fastest plain pass over the same planes in this run" % (hbm_gbs, rates["ceiling"])
    else:
        roofline = {"bound": "valu", "achieved": useful_tflops, "peak": FP32_VALU_PLAIN_TFLOPS, "unit": "TFLOP/s",
                    "frac": useful_tflops / FP32_VALU_PLAIN_TFLOPS, "traffic": dom_bytes,
                    "useful_valu_frac": useful_tflops / FP32_VALU_PLAIN_TFLOPS, "staged_valu_frac": staged_tflops / FP32_VALU_PLAIN_TFLOPS,
                    "flops_per_cell_step": ops, "staged_cells_per_launch": staged_cells,
                    "peak_basis": "256 compute units x 64 lanes x 2.4 GHz, one add or multiply per lane and clock (no FMA: results must round as "
                                  "the un-fused program's; no packed fp32 on this pool)",
                    "vector_alu_busy": t_dom["vector_alu_busy"] if t_dom else None,
                    "hbm": hbm,
                    "limiter": "vector ALUs: a time-fused launch advances %d steps per byte it moves, so its stencil arithmetic sets its duration "
                               "(%.2f of the plain VALU rate on the cells of the domain, %.2f with the halo and stale cells it also computes); "
                               "its HBM traffic runs at %.0f GB/s against %.0f GB/s for the fastest plain pass over the same planes in this run "
                               "(vendor device-to-device copy: %.0f GB/s)"
                               % (fused_steps, useful_tflops / FP32_VALU_PLAIN_TFLOPS, staged_tflops / FP32_VALU_PLAIN_TFLOPS, hbm_gbs, rates["ceiling"], rates["vendor_d2d"])}
    roofline.update({"kernel": dom[0], "kernel_ms": dom[1][0], "launches_per_step": dom[1][1],
                     "time_steps_per_launch": fused_steps, "cells_per_launch": cells})
    out = {
        "value": call_bytes / (ms * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": ms, "warmup_extra_steps": EXTRA_WARMUP.get("last", 0),
        "value_basis": "HBM bytes moved per call (hardware counters per kernel x launches%s) / time per call"
                       % ("" if all(measured.values()) else "; read-once-write-once minimum for kernels without a counter record of their present source"),
        "value_lower_bound_gbs": sum(minimum[k] * v[1] for k, v in prof.items()) / (ms * 1e-3) / 1e9,
        "value_lower_bound_basis": "needs no counters: every launch reads one plane and writes each plane it leaves once",
        "algorithmic_gbs": alg_bytes / (ms * 1e-3) / 1e9,
        "algorithmic_basis": "8 bytes per cell and time step of the un-fused program (32 x 2 x 8192^2 x 4 B = 17.18 GB per call)",
        "roofline": roofline,
        "streaming_rates_gbs": rates,
        "kernels": {k: {"ms": v[0], "launches_per_step": v[1], "traffic": measured[k]["bytes"] if measured[k] else None} for k, v in prof.items()},
    }
    if with_cpu:
        cpu = runtime.Program(oracle_build.cpu_program_library(PROGRAMS, name), name, needs_gpu_runtime=False)
        host = planes.copy()
        sec, runs = cpu_time(lambda: cpu(host))
        out["cpu_baseline"] = {"value": alg_bytes / sec / 1e9, "unit": "GB/s", "cores": cpu_threads(), "kind": "port",
                               "sample": "whole workload (8192x8192, 32 steps), median of %d runs of the CPU-generated "
                                         "code (parallelize y, vectorize x by 8; g++ -O2 -mavx, OpenMP); bytes = 8 per cell and "
                                         "time step, which is what the un-fused CPU code moves" % runs}
    return out


def bench_sgemm(M, steps, warmup, with_cpu):
    from tiramisu_amd import runtime
    from oracle import build as oracle_build
    N = K = M
    name = "sgemm_%dx%dx%d" % (M, N, K)
    rng = np.random.RandomState(M)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    C = np.zeros((M, N), np.float32)
    scal = np.array([1.0, 0.0], np.float32)
    dA, dB, dC = device_array(A), device_array(B), device_array(C)
    prog = runtime.load(PROGRAMS, name)
    args = (scal, dA.buffer(), dB.buffer(), dC.buffer())
    ms = time_steps(lambda: prog(*args), steps, warmup)
    flop = 2.0 * M * N * K
    prof = kernel_profile(lambda: prog(*args), steps)
    dom = max(prof.items(), key=lambda kv: kv[1][0] * kv[1][1])
    kernel_ms, basis = launch_duration(prof, dom[0], ms)
    achieved = flop / (kernel_ms * 1e-3) / 1e12
    out = {
        "value": flop / (ms * 1e-3) / 1e9, "unit": "GFLOP/s", "ms_per_step": ms, "warmup_extra_steps": EXTRA_WARMUP.get("last", 0),
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / FP32_MFMA_PEAK_TFLOPS, "traffic": (kernel_traffic(name, dom[0]) or {}).get("bytes"),
                     "kernel": dom[0], "kernel_ms": kernel_ms, "kernel_ms_basis": basis, "kernel_ms_between_events": dom[1][0],
                     "frac_between_events": flop / (dom[1][0] * 1e-3) / 1e12 / FP32_MFMA_PEAK_TFLOPS},
    }
    if with_cpu:
        cpu = runtime.Program(oracle_build.cpu_program_library(PROGRAMS, name), name, needs_gpu_runtime=False)
        Ch = C.copy()
        sec, runs = cpu_time(lambda: cpu(scal, A, B, Ch), min_seconds=2.0, max_runs=3)
        out["cpu_baseline"] = {"value": flop / sec / 1e9, "unit": "GFLOP/s", "cores": cpu_threads(), "kind": "port",
                               "sample": "whole workload (%d^3), median of %d runs of the CPU-generated code "
                                         "(parallelize i, vectorize j by 8)" % (M, runs)}
    for d in (dA, dB, dC):
        d.free()
    return out


SKIP_STREAMING_RATES = False   # --no-streaming-rates: counter runs want the workload's own kernels only


def streaming_rates(reps=30, with_torch=False):
    """Read-once-write-once rates on the benchmark's plane size (256 MiB read + 256 MiB written per pass, GB/s of both
    directions together), measured here: the ceiling that the HBM-bound stencil launches are stated against.
      vendor_d2d          hipMemcpyAsync device to device (through the runtime ABI's tiramisu_hip_memcpy_device_to_device)
      copy_plane          the copy program on the schedule-faithful emitter (4 bytes per lane)
      copy_plane_quads    the same program taken by the stencil emitter (16 bytes per lane, non-temporal stores)
      torch_copy / torch_add   torch.Tensor.copy_ and an element-wise add (second opinions; only with `with_torch`)"""
    from tiramisu_amd import runtime
    if SKIP_STREAMING_RATES:
        return {"ceiling": float("nan"), "vendor_d2d": float("nan"), "ceiling_basis": "not measured (--no-streaming-rates)"}
    w = runtime.wrappers()
    n = 8192
    nbytes = 2.0 * n * n * 4
    a = np.ones((n, n), np.float32)
    dS, dD = device_array(a), device_array(a)
    out = {}

    def rate(call):
        for _ in range(reps):
            call()
        w.tiramisu_hip_stream_synchronize(0)
        best = None
        for _ in range(3):
            with runtime.DeviceTimer() as t:
                for _ in range(reps):
                    call()
            best = t.ms if best is None else min(best, t.ms)
        return nbytes / (best / reps * 1e-3) / 1e9
    out["vendor_d2d"] = rate(lambda: w.tiramisu_hip_memcpy_device_to_device(dD.ptr, dS.ptr, n * n * 4))
    for prog_name in ("copy_plane", "copy_plane_quads"):
        prog = runtime.load(PROGRAMS, prog_name)
        args = (dS.buffer(), dD.buffer())
        out[prog_name] = rate(lambda: prog(*args))
    dS.free()
    dD.free()
    if with_torch:
        try:
            import torch
            ta = torch.ones(n, n, device="cuda")
            tb = torch.empty_like(ta)
            for key, call in (("torch_copy", lambda: tb.copy_(ta)), ("torch_add", lambda: torch.add(ta, 1.0, out=tb))):
                for _ in range(reps):
                    call()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(reps):
                    call()
                e1.record()
                torch.cuda.synchronize()
                out[key] = nbytes / (e0.elapsed_time(e1) / reps * 1e-3) / 1e9
        except ImportError:
            pass
    out["ceiling"] = max(out.values())
    out["ceiling_basis"] = "the fastest of these passes over 256 MiB in + 256 MiB out, timed in this run: " + ", ".join(k for k in out if k != "ceiling")
    return out


def bench_copy(steps, warmup, with_cpu):
    """Streaming calibration: 256 MiB -> 256 MiB by the vendor's device-to-device copy, by torch, and by the copy
    program on both emitters.  `value` is the copy program as the back-end compiles it when left alone."""
    from tiramisu_amd import runtime
    n = 8192
    a = np.ones((n, n), np.float32)
    dS, dD = device_array(a), device_array(a)
    prog = runtime.load(PROGRAMS, "copy_plane_quads")
    args = (dS.buffer(), dD.buffer())
    ms = time_steps(lambda: prog(*args), steps, warmup)
    nbytes = 2.0 * n * n * 4
    dS.free()
    dD.free()
    rates = streaming_rates(max(steps, 20), with_torch=True)
    out = {"value": nbytes / (ms * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": ms, "warmup_extra_steps": EXTRA_WARMUP.get("last", 0),
           "roofline": {"bound": "hbm", "achieved": nbytes / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": nbytes, "kernel": "copy_plane_quads"},
           "streaming_rates_gbs": rates}
    return out


def bench_sweep5(steps, warmup, with_cpu):
    """One 5-point sweep out of place on 8192 x 8192 floats (programs/stencil_sweep.cpp): the stencil back-end's
    single-step form.  Bytes: the plane read once and written once."""
    from tiramisu_amd import runtime
    n = 8192
    rng = np.random.RandomState(3)
    dS, dD = device_array(rng.uniform(0, 1, (n, n)).astype(np.float32)), device_array(np.zeros((n, n), np.float32))
    prog = runtime.load(PROGRAMS, "sweep5_8192x8192")
    args = (dS.buffer(), dD.buffer())
    ms = time_steps(lambda: prog(*args), steps, warmup)
    prof = kernel_profile(lambda: prog(*args), steps)
    dom = max(prof.items(), key=lambda kv: kv[1][0] * kv[1][1])
    nbytes = 2.0 * n * n * 4
    dS.free()
    dD.free()
    rates = streaming_rates()
    achieved = nbytes / (dom[1][0] * 1e-3) / 1e9
    out = {"value": nbytes / (ms * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": ms, "warmup_extra_steps": EXTRA_WARMUP.get("last", 0),
           "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": achieved / HBM_PEAK_GBS, "traffic": (kernel_traffic("sweep5_8192x8192", dom[0]) or {}).get("bytes"),
                        "kernel": dom[0], "kernel_ms": dom[1][0],
                        "streaming_ceiling_gbs": rates["ceiling"], "frac_of_streaming_ceiling": achieved / rates["ceiling"],
                        "limiter": "hbm: %.0f GB/s against %.0f GB/s for the fastest plain pass over the same planes in this run (vendor "
                                   "device-to-device copy %.0f GB/s)" % (achieved, rates["ceiling"], rates["vendor_d2d"])},
           "streaming_rates_gbs": rates}
    return out


def _generic_bench(name, host_arrays, flop, peak_tflops, steps, warmup, with_cpu, cpu_sample, dominant_flop_share=1.0):
    """A compiled function whose arguments are all GPU-resident (except leading host scalars)."""
    from tiramisu_amd import runtime
    from oracle import build as oracle_build
    devs, args = [], []
    for a in host_arrays:
        if isinstance(a, tuple):         # ("host", array): passed as a host buffer
            args.append(a[1])
        else:
            d = device_array(a)
            devs.append(d)
            args.append(d.buffer())
    prog = runtime.load(PROGRAMS, name)
    ms = time_steps(lambda: prog(*args), steps, warmup)
    prof = kernel_profile(lambda: prog(*args), max(1, min(steps, 5)))
    dom = max(prof.items(), key=lambda kv: kv[1][0] * kv[1][1])
    dom_flop = flop * dominant_flop_share / dom[1][1]   # flops of an average launch of the dominant kernel
    kernel_ms, basis = launch_duration(prof, dom[0], ms)
    achieved = dom_flop / (kernel_ms * 1e-3) / 1e12
    out = {"value": flop / (ms * 1e-3) / 1e9, "unit": "GFLOP/s", "ms_per_step": ms, "warmup_extra_steps": EXTRA_WARMUP.get("last", 0),
           "roofline": {"bound": "mfma", "achieved": achieved, "peak": peak_tflops, "unit": "TFLOP/s",
                        "frac": achieved / peak_tflops, "traffic": (kernel_traffic(name, dom[0]) or {}).get("bytes"),
                        "kernel": dom[0], "kernel_ms": kernel_ms, "kernel_ms_basis": basis, "kernel_ms_between_events": dom[1][0],
                        "frac_between_events": dom_flop / (dom[1][0] * 1e-3) / 1e12 / peak_tflops,
                        "launches_per_step": dom[1][1]},
           "kernels": {k: {"ms": v[0], "launches_per_step": v[1]} for k, v in prof.items()}}
    if with_cpu:
        cpu = runtime.Program(oracle_build.cpu_program_library(PROGRAMS, name), name, needs_gpu_runtime=False)
        host = [a[1] if isinstance(a, tuple) else a.copy() for a in host_arrays]
        sec, runs = cpu_time(lambda: cpu(*host), min_seconds=2.0, max_runs=3)
        out["cpu_baseline"] = {"value": flop / sec / 1e9, "unit": "GFLOP/s", "cores": cpu_threads(), "kind": "port",
                               "sample": "whole workload, median of %d run(s) of the CPU-generated code (%s)" % (runs, cpu_sample)}
    for d in devs:
        d.free()
    return out


def bench_sgemm_bf16(steps, warmup, with_cpu):
    M = N = K = 4096
    rng = np.random.RandomState(16)

    def bf16(a):
        u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
        return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    A, B = bf16(rng.uniform(-1, 1, (M, K))), bf16(rng.uniform(-1, 1, (K, N)))
    C = np.zeros((M, N), np.float32)
    return _generic_bench("sgemm_bf16_4096x4096x4096", [("host", np.array([1.0, 0.0], np.float32)), A, B, C],
                          2.0 * M * N * K, BF16_MFMA_PEAK_TFLOPS, steps, warmup, with_cpu,
                          "parallelize i, vectorize j by 8; bf16 operands widened to fp32 on load -- the reference has no bf16 type")


def bench_conv2d(steps, warmup, with_cpu):
    N, CI, CO, H = 32, 64, 64, 112
    rng = np.random.RandomState(4)
    xp = np.zeros((N, CI, H + 2, H + 2), np.float32)
    xp[:, :, 1:-1, 1:-1] = rng.uniform(0, 1, (N, CI, H, H)).astype(np.float32)
    w = rng.uniform(-0.1, 0.1, (CO, CI, 3, 3)).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, (CO,)).astype(np.float32)
    out = np.zeros((N, CO, H, H), np.float32)
    return _generic_bench("conv2d_32x64x64x112", [xp, w, b, out], 2.0 * N * CO * H * H * CI * 9, FP32_MFMA_PEAK_TFLOPS,
                          steps, warmup, with_cpu, "parallelize n, vectorize x by 8")


def bench_lstm(steps, warmup, with_cpu):
    L, B, H, S = 4, 64, 512, 100
    rng = np.random.RandomState(5)
    w = rng.uniform(-0.08, 0.08, (L, 2, 4 * H, H)).astype(np.float32)
    b = rng.uniform(-0.08, 0.08, (L, 4 * H)).astype(np.float32)
    x = rng.uniform(-1, 1, (S, B, H)).astype(np.float32)
    y = np.zeros((S, B, H), np.float32)
    flop = L * S * 2 * (2.0 * B * 4 * H * H)
    return _generic_bench("lstm_4x64x512x100", [w, b, x, y], flop, FP32_MFMA_PEAK_TFLOPS, steps, warmup,
                          with_cpu, "naive ordered nest, no tiling, parallelize(k): the reference's cpu/generator.cpp order")   # one kernel does all the flops: the fused cell


def bench_sgemm_cache_shared(steps, warmup, with_cpu):
    """The reference's tuned cache_shared schedule (generator3) at 3072^3, kept on the schedule-faithful
    emitter: VALU FMAs fed from LDS tiles.  Not one of the benchmark configurations and not part of
    `--workload all`; it is here so that the emitter's LDS behaviour can be put under the profiler."""
    M = N = K = 3072
    rng = np.random.RandomState(30)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    C = np.zeros((M, N), np.float32)
    out = _generic_bench("sgemm_cache_shared_3072", [("host", np.array([1.0, 0.0], np.float32)), A, B, C],
                         2.0 * M * N * K, FP32_VALU_PEAK_TFLOPS, steps, warmup, False, "")
    out["roofline"]["bound"] = "valu"
    return out


WORKLOADS = {
    "heat2d": lambda s, w, c: bench_heat2d(s, w, c),
    "sgemm1024": lambda s, w, c: bench_sgemm(1024, s, w, c),
    "sgemm4096": lambda s, w, c: bench_sgemm(4096, s, w, c),
    "sgemm4096_bf16": bench_sgemm_bf16,
    "conv2d": bench_conv2d,
    "lstm": bench_lstm,
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="all")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-streaming-rates", action="store_true", help="skip the copy passes that calibrate the streaming ceiling")
    a = ap.parse_args()
    global SKIP_STREAMING_RATES
    SKIP_STREAMING_RATES = a.no_streaming_rates
    if a.gpus != 1:
        sys.exit("bench.py measures one GPU: this back-end compiles single-GPU Tiramisu programs and nothing here "
                 "uses a second device (run with --gpus 1)")
    from tiramisu_amd import runtime
    if runtime.wrappers().tiramisu_hip_device_count() < 1:
        sys.exit("no HIP device visible")
    WORKLOADS["copy"] = bench_copy   # calibration only, not part of "all"
    WORKLOADS["sweep5"] = bench_sweep5   # the single-step form of the stencil back-end, not part of "all"
    WORKLOADS["sgemm_cache_shared"] = bench_sgemm_cache_shared   # profiling of the schedule-faithful emitter only
    names = [n for n in WORKLOADS if n not in ("copy", "sweep5", "sgemm_cache_shared")] if a.workload == "all" else [a.workload]
    results = {}
    for n in names:
        with_cpu = not a.no_cpu
        results[n] = WORKLOADS[n](a.steps, a.warmup, with_cpu)
    head_name = "heat2d" if "heat2d" in results else names[0]
    head = results[head_name]
    line = {
        "metric": "GFLOP/s (sgemm, conv2d, LSTM) + HBM GB/s (heat2d), % of roofline, 1 GPU",
        "value": head["value"], "unit": head["unit"], "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if head_name == "sgemm4096_bf16" else "f32", "warmup_extra_steps": head.get("warmup_extra_steps", 0),
        "data": "synthetic (seeded uniform inputs, already resident in HBM)",
        "config": {"workload": {"heat2d": "heat2d 5-point stencil, fp32 grid 8192x8192, 32 time steps (benchmark configs[1])",
                                "sgemm1024": "sgemm fp32 1024^3 (benchmark configs[0])",
                                "sgemm4096": "sgemm fp32 4096^3 (benchmark configs[2])",
                                "sgemm4096_bf16": "sgemm bf16-in/fp32-acc 4096^3 (benchmark configs[2], bf16 variant)",
                                "conv2d": "conv2d+bias+ReLU N32 C64->64 112x112 3x3 (benchmark configs[3])",
                                "lstm": "4-layer LSTM B64 H512 S100 (benchmark configs[4])"}.get(head_name, head_name)},
        "roofline": head["roofline"],
        "cpu_baseline": head.get("cpu_baseline"),
        **{k: head[k] for k in ("value_basis", "value_lower_bound_gbs", "value_lower_bound_basis", "algorithmic_gbs", "algorithmic_basis", "streaming_rates_gbs") if k in head},
        "workloads": {k: v for k, v in results.items() if k != head_name},
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
