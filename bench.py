#!/usr/bin/env python3
"""Headline benchmark: p=3 sum-factorised hex mass-operator apply, fp64, 2^18 elements, one MI355X.

A step is one fused multi-kernel launch (7 contractions, X -> Y) over all elements with every tensor already
resident in HBM.  Prints ONE JSON line:

  value           GDOF/s over the timed steps, host-side TensorEngine overhead included (wall clock between two
                  device synchronisations)
  roofline        algorithmic bytes of one launch (X + D + Y = 2024 B per element) over the launch duration
                  measured with HIP events on the library's stream, against the 8 TB/s HBM peak; `traffic` is the
                  HBM traffic that hardware counters showed for exactly the kernel that ran (identified by name and
                  a hash of its generated source), null for any other kernel
  cpu_baseline    the same chain on the host: the reference's own CPUInterpreted executor (oracle/_ref, kind
                  "reference") or, if that library is absent, the plain-C restatement (kind "port"), one thread,
                  on a bounded sample of elements
  store_all       the same launch when the six intermediates are ordinary (non-transient) tensors, i.e. also
                  written to HBM as the reference's generated kernel always does: what a caller gets who changes
                  nothing but the policy string
  all_configs     the other four baseline configurations at their full sizes, each with launch time by HIP
                  events, algorithmic GB/s, fraction of the HBM peak, GFLOP/s and its own single-thread CPU
                  baseline (on a stated sample where the host would take minutes)
"""
import argparse
import hashlib
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
ONLY_ROTATED = False   # --only-rotated
METRIC = "GDOF/s + % HBM peak, p=3 sum-factorised hex mass apply fp64 (1 GPU)"

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (each scaled by what the same counter
# reads for a copy kernel of known size), keyed by the kernel the counters were taken on: (name of its first
# function, first 16 hex digits of the SHA-1 of the generated source).  A generator change that alters the source of
# a kernel therefore drops its figure (the line then says null) until the counters are taken again.
TRAFFIC_BY_KERNEL = {
    ("acro_mk_4ceea56515f0c53c", "5b2c83c4dcb5398d"): 547273919,            # cfg4, intermediates transient
    ("acro_mk_664cf228dc3d274e", "bb5ff2ad54f2a970"): 1815902982,           # cfg4, every intermediate stored
    ("acro_red_35ac69981569e511_partial", "1698cfe138e16625"): 83943091,    # cfg1 (first of its two launches)
    ("batchMatrixKernel<3,inv,det>", "c901ed174aa3fd9b"): 637556292,        # cfg2 (precompiled: hash of hip_ops.hip)
    ("acro_mk_567e3a4d341f4dc2", "663c472f29b65c65"): 210806499,            # cfg3
    ("acro_mk_e688ac87da28a7bd", "018c1f37edc57625"): 5258904464,           # cfg5
    ("scatterKernel2", "c901ed174aa3fd9b"): 261111812,                      # node vector -> element vector
    ("sumGatherKernel", "c901ed174aa3fd9b"): 295431127,                     # element vector -> node vector
    ("acro_mk_e5e3c68e773e2587", "2f278ec4d44c8ab3"): 2517052766,           # geometric factors from the Jacobians, one launch
    ("acro_mk_ff9b33d31033d4fa", "01c28d4e15a8863a"): 547324322,            # scatter read through the map by the mass apply
}


def kernel_identity(engine, precompiled=None):
    """(function names, source hash) of the kernel(s) the engine's most recent launch used.  `precompiled` names a
    kernel of the library itself (the batched small-matrix and index operations): its source is hip_ops.hip."""
    if precompiled is not None:
        with open(os.path.join(ROOT, "acrotensor_amd", "csrc", "hip_ops.hip"), "rb") as f:
            return [precompiled], hashlib.sha1(f.read()).hexdigest()[:16]
    src = engine.GetLastImplementation()
    names = re.findall(r"__global__[^\n]*?\bvoid\s+(\w+)\s*\(", src)
    return names, hashlib.sha1(src.encode()).hexdigest()[:16]


def measured_traffic(engine, precompiled=None):
    names, digest = kernel_identity(engine, precompiled)
    return TRAFFIC_BY_KERNEL.get((names[0] if names else "", digest))


def settle_clocks(at, workloads, wl, engine, tensors, seconds):
    """Untimed launches before the warm-up: the first ~20 ms of sustained load run through a power-management
    transient (boost clocks, then a clamp, then the sustainable state); measurements start after it."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(100):
            workloads.launch(wl, engine, tensors)
        at.synchronize()


def time_steps(at, workloads, wl, engine, tensors, steps, warmup):
    for _ in range(warmup):
        workloads.launch(wl, engine, tensors)
    at.synchronize()
    t0 = time.perf_counter()
    with at.hip_event_timer() as ev:
        for _ in range(steps):
            workloads.launch(wl, engine, tensors)
    at.synchronize()
    wall = time.perf_counter() - t0
    return wall, ev.ms * 1e-3


def time_steps_rotating(at, workloads, wl, engine, sets, steps, warmup):
    """`steps` launches issued round-robin over the buffer sets."""
    n = len(sets)
    for i in range(max(n, warmup)):
        workloads.launch(wl, engine, sets[i % n])
    at.synchronize()
    t0 = time.perf_counter()
    with at.hip_event_timer() as ev:
        for i in range(steps):
            workloads.launch(wl, engine, sets[i % n])
    at.synchronize()
    wall = time.perf_counter() - t0
    return wall, ev.ms * 1e-3


def host_checker():
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle  # tests/oracle.py - checker access, used here only for the reported CPU baselines

    if oracle.have_reference():
        return oracle.Reference(), "reference"
    return oracle.Oracle(), "port"


def cpu_baseline(workloads, sample_elems):
    checker, kind = host_checker()
    wl = workloads.config4(E=sample_elems)
    t0 = time.perf_counter()
    workloads.run_on_checker(wl, checker)
    dt = time.perf_counter() - t0
    return {
        "value": wl.dof / dt * 1e-9,
        "unit": "GDOF/s",
        "cores": 1,
        "kind": kind,
        "sample": "%d of 262144 elements, whole 7-kernel chain, one pass, %.1f s" % (sample_elems, dt),
    }


def cpu_baseline_for(name, workloads):
    """Single-thread host figure for one of the other baseline configurations, in the unit of its GPU line."""
    checker, kind = host_checker()
    if name == "cfg1":
        wl = workloads.config1()
        passes = 25
        t0 = time.perf_counter()
        for _ in range(passes):
            workloads.run_on_checker(wl, checker)
        dt = (time.perf_counter() - t0) / passes
        value, unit, sample = wl.algorithmic_bytes / dt * 1e-9, "GB/s", "all 1048576 slices, mean of %d passes of %.3f s" % (passes, dt)
    elif name == "cfg2":
        J = workloads.config2_inputs()
        passes = 25
        t0 = time.perf_counter()
        for _ in range(passes):
            checker.batch_matrix_inv_det(J)
        dt = (time.perf_counter() - t0) / passes
        value, unit, sample = J.shape[0] * J.shape[1] / dt * 1e-9, "Gmatrices/s", "all 4194304 matrices, mean of %d passes of %.3f s" % (passes, dt)
    elif name == "cfg3":
        n = 16384
        wl = workloads.config3(E=n)
        t0 = time.perf_counter()
        workloads.run_on_checker(wl, checker)
        dt = time.perf_counter() - t0
        value, unit, sample = wl.algorithmic_bytes / dt * 1e-9, "GB/s", "%d of 32768 elements, kernel as written, one pass, %.1f s" % (n, dt)
    elif name == "cfg5":
        n = 8192
        wl = workloads.config5(E=n)
        t0 = time.perf_counter()
        workloads.run_on_checker(wl, checker)
        dt = time.perf_counter() - t0
        value, unit, sample = wl.dof / dt * 1e-9, "GDOF/s", "%d of 65536 elements, whole 18-kernel chain, one pass, %.1f s" % (n, dt)
    else:
        raise ValueError(name)
    return {"value": value, "unit": unit, "cores": 1, "kind": kind, "sample": sample}


FP64_PEAK_GFLOPS = 78600.0

_MEMO = {}


def memo(fn, *args):
    """Host arrays and workloads are generated once and shared by the buffer sets of a rotated measurement (they are
    only ever copied from)."""
    key = (fn.__name__,) + args
    if key not in _MEMO:
        _MEMO[key] = fn(*args)
    return _MEMO[key]


def sets_beyond_the_last_level_cache(abytes, requested=0):
    """Number of buffer sets to rotate over so that a set's data cannot survive in the 256 MB memory-side cache
    between two launches on it: together the sets exceed 1 GiB; a launch that moves 2 GiB or more needs no second
    set.  `requested` > 0 overrides."""
    if requested > 0:
        return requested
    if abytes >= (2 << 30):
        return 1
    return min(32, (1 << 30) // abytes + 1)


# Single kernels a user of the reference's API writes, at large batch sizes: (kernel, input shapes, output shape).
KERNEL_SHAPES = [
    ("A_e_i = B_e_i", [(1 << 22, 16)], (1 << 22, 16)),
    ("A_e_i += B_e_i", [(1 << 22, 16)], (1 << 22, 16)),
    ("A_e_i = B_e_i C_e_i D_e_i", [(1 << 22, 16)] * 3, (1 << 22, 16)),
    ("A_e_i = B_e_i_j C_j", [(1 << 20, 8, 8), (8,)], (1 << 20, 8)),
    ("A_e_i = B_e_i_j C_e_j", [(1 << 20, 8, 8), (1 << 20, 8)], (1 << 20, 8)),
    ("A_e_i = B_e_i_j C_e_j", [(1 << 18, 16, 16), (1 << 18, 16)], (1 << 18, 16)),
    ("A_e_i = B_e_i_j C_e_j", [(1 << 17, 27, 27), (1 << 17, 27)], (1 << 17, 27)),
    ("A_e_i = B_e_i_j C_e_j", [(1 << 15, 64, 64), (1 << 15, 64)], (1 << 15, 64)),
    ("A_e_i_k = B_e_i_j C_e_j_k", [(1 << 21, 3, 3), (1 << 21, 3, 3)], (1 << 21, 3, 3)),
    ("A_e_i_k = B_e_i_j C_e_j_k", [(1 << 20, 4, 4), (1 << 20, 4, 4)], (1 << 20, 4, 4)),
    ("A_e_i_k = B_e_i_j C_e_j_k", [(1 << 18, 8, 8), (1 << 18, 8, 8)], (1 << 18, 8, 8)),
    ("A_e_i_k = B_e_i_j C_j_k", [(1 << 20, 8, 8), (8, 8)], (1 << 20, 8, 8)),
    ("A_e = B_e_i C_e_i", [(1 << 21, 16), (1 << 21, 16)], (1 << 21,)),
    ("A_e = B_e_n", [(1 << 16, 1024)], (1 << 16,)),
    ("A_e_i = B_e_i_n", [(1 << 17, 4, 256)], (1 << 17, 4)),
    ("A_e_i_j = B_e_i C_e_j", [(1 << 20, 8), (1 << 20, 8)], (1 << 20, 8, 8)),
    ("A_e_i_j = B_e_j_i", [(1 << 20, 8, 8)], (1 << 20, 8, 8)),
    ("A_e_i_j_k = B_e_k_j_i", [(1 << 16, 8, 8, 8)], (1 << 16, 8, 8, 8)),
    ("A_e_i = B_e_i_i", [(1 << 20, 8, 8)], (1 << 20, 8)),
    ("A_e_q_j_k = B_q_i X_e_i_j_k", [(5, 4), (1 << 19, 4, 4, 4)], (1 << 19, 5, 4, 4)),
    ("A_e_i = B_i_j X_e_j", [(64, 64), (1 << 18, 64)], (1 << 18, 64)),
    ("U_e_q = B_q_i X_e_i", [(125, 64), (1 << 17, 64)], (1 << 17, 125)),
    ("A_e_i_k = B_i_j X_e_j_k", [(64, 64), (1 << 16, 64, 3)], (1 << 16, 64, 3)),
    ("A_e_i_k = B_i_j X_e_j_k", [(16, 16), (1 << 18, 16, 3)], (1 << 18, 16, 3)),
    ("A_e_i = B_i_j X_e_j", [(7, 9), (1 << 21, 9)], (1 << 21, 7)),
    ("A_e_i = B_i_j X_e_j", [(20, 5), (1 << 21, 5)], (1 << 21, 20)),
    ("A_e_i = B_i_j X_e_j", [(27, 3), (1 << 21, 3)], (1 << 21, 27)),
    ("A_e_i = B_i_j X_e_j", [(27, 27), (1 << 19, 27)], (1 << 19, 27)),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(1 << 16, 16, 16), (1 << 16, 16, 16)], (1 << 16, 16, 16)),
    ("A_e_i_j = B_e_i_k C_e_j_k", [(1 << 14, 32, 32), (1 << 14, 32, 32)], (1 << 14, 32, 32)),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(29127, 24, 24), (29127, 24, 24)], (29127, 24, 24)),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(138654, 11, 11), (138654, 11, 11)], (138654, 11, 11)),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(26843, 25, 25), (26843, 25, 25)], (26843, 25, 25)),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(10485, 40, 40), (10485, 40, 40)], (10485, 40, 40)),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(15406, 33, 33), (15406, 33, 33)], (15406, 33, 33)),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(12255, 37, 37), (12255, 37, 37)], (12255, 37, 37)),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(7281, 48, 48), (7281, 48, 48)], (7281, 48, 48)),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(5972, 53, 53), (5972, 53, 53)], (5972, 53, 53)),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(5546, 55, 55), (5546, 55, 55)], (5546, 55, 55)),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(4227, 63, 63), (4227, 63, 63)], (4227, 63, 63)),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(4096, 64, 64), (4096, 64, 64)], (4096, 64, 64)),
    ("A_e_i_j = B_e_i_k C_e_j_k", [(4096, 64, 64), (4096, 64, 64)], (4096, 64, 64)),
    # larger element matrices and a plain matrix product: tiles on the FP64 matrix cores (the last one is bound by
    # arithmetic; its fraction of the FP64 peak is in `frac_fp64_cold`)
    ("A_e_i_j = B_e_i_k C_e_k_j", [(2730, 80, 80), (2730, 80, 80)], (2730, 80, 80)),
    ("A_e_i_j = B_e_i_k C_e_k_j", [(1024, 128, 128), (1024, 128, 128)], (1024, 128, 128)),
    ("A_i_j = B_i_k C_k_j", [(2048, 2048), (2048, 2048)], (2048, 2048)),
    ("A_i = C_i_j B_j", [(1 << 20, 64), (64,)], (1 << 20,)),
    ("M_e_i1_i2_j1_j2 = B_k1_i1 B_k1_j1 B_k2_i2 B_k2_j2 D_e_k1_k2", [(5, 4)] * 4 + [(1 << 19, 5, 5)], (1 << 19, 4, 4, 4, 4)),
    ("A_i_j = B_j_i", [(1 << 22, 16)], (16, 1 << 22)),
    ("S_i = A_n_i", [(1 << 20, 64)], (64,)),
    ("S_i = A_i_n", [(64, 1 << 20)], (64,)),
    ("S_i_j = A_e_i_j", [(1 << 17, 32, 32)], (32, 32)),
    ("A_i_j = B_j_i", [(8192, 8192)], (8192, 8192)),
    ("A_i_j = B_e_i C_e_j", [(1 << 21, 32), (1 << 21, 32)], (32, 32)),
    ("A_i_j = B_e_i C_e_j", [(1 << 20, 64), (1 << 20, 64)], (64, 64)),
    ("A_e = B_e_i_j C_i D_j", [(1 << 20, 8, 8), (8,), (8,)], (1 << 20,)),
    ("A_i_e = B_i_e C_i_e", [(16, 1 << 22), (16, 1 << 22)], (16, 1 << 22)),
    ("G_e_d_q = D_d_q_i X_e_i", [(3, 64, 64), (1 << 18, 64)], (1 << 18, 3, 64)),
    ("A_e_i = B_i_j X_e_j", [(81, 8), (1 << 20, 8)], (1 << 20, 81)),
    ("Y_e_i_j = B_q_i B_r_j D_e_q_r U_e_q_r", [(5, 4), (5, 4), (1 << 20, 5, 5), (1 << 20, 5, 5)], (1 << 20, 4, 4)),
    ("U_e_q_r_s = B_q_i B_r_j B_s_k X_e_i_j_k", [(5, 4), (5, 4), (5, 4), (1 << 18, 4, 4, 4)], (1 << 18, 5, 5, 5)),
    # a gradient at a point: three rows applied to vectors of 32 values
    ("G_e_d = D_d_i X_e_i", [(3, 32), (1 << 20, 32)], (1 << 20, 3)),
    # short sums per entry (products into an LDS tile, then a lane per sum)
    ("A_e = B_e_i", [(1 << 22, 9)], (1 << 22,)),
    ("A_e = B_e_i C_e_i", [(1 << 20, 27), (1 << 20, 27)], (1 << 20,)),
    # operands that carry a contraction index alone are summed first
    ("A_e = B_e_j C_e_i", [(1 << 20, 32), (1 << 20, 27)], (1 << 20,)),
    # a long contraction that no other schedule takes: shared out over workgroups by rows
    ("A_e += B_i C_e_i", [(8192,), (4096, 8192)], (4096,)),
]


def schedule_line(source):
    """The first line of the schedule comment of a generated kernel (after "// Generated by ...", past notes in
    brackets)."""
    lines = source.splitlines()
    for i, line in enumerate(lines):
        if line.startswith("// Generated by"):
            rest = [l for l in lines[i + 1:i + 4] if not l.startswith("// (")]
            return rest[0][3:] if rest else ""
    return ""


def flops_as_written(kernel, in_shapes, out_shape):
    """Arithmetic of a contraction of two factors: a multiplication and an addition per combination of index values;
    0 for a kernel without a contracted index and for one with more factors."""
    lhs, rhs = kernel.replace("+=", "=").replace("-=", "=").split("=")
    extent = {}
    for token, shape in zip([lhs.split()[0]] + rhs.split(), [out_shape] + list(in_shapes)):
        for name, n in zip(token.split("_")[1:], shape):
            extent[name] = n
    if not set(extent) - set(lhs.split()[0].split("_")[1:]) or len(rhs.split()) != 2:
        return 0                                       # (more than two factors: the generator sums in steps, far fewer operations)
    terms = 1
    for n in extent.values():
        terms *= n
    return terms * len(rhs.split())


def kernel_shapes(at, args):
    """One line for the whole list: per kernel the launch time by HIP events and algorithmic bytes / time against the
    HBM peak, re-launched on one set of tensors (`frac`) and round-robin over enough sets to exceed 1 GiB
    (`frac_cold`); `value` is the geometric mean of the cold fractions."""
    import math
    import numpy as np
    t_start = time.perf_counter()
    engine = at.TensorEngine("HIP")
    steps = min(args.steps, 20)
    results = []
    for kernel, in_shapes, out_shape in KERNEL_SHAPES:
        abytes = sum(int(np.prod(s)) * 8 for s in in_shapes) + int(np.prod(out_shape)) * 8 * (2 if "+=" in kernel else 1)
        n_sets = sets_beyond_the_last_level_cache(abytes, args.rotate)
        sets = []
        for _ in range(n_sets):
            tensors = [at.Tensor(*s) for s in in_shapes] + [at.Tensor(*out_shape)]
            for t in tensors:
                t.SwitchToGPU()
                t.Set(0.5)
            sets.append(tensors)
        step = lambda i=0: engine(kernel, sets[i][-1], *sets[i][:-1])
        same = (lambda k: k % n_sets) if ONLY_ROTATED else (lambda k: 0)
        for k in range(5):
            step(same(k))
        at.synchronize()
        with at.hip_event_timer() as ev:
            for k in range(steps):
                step(same(k))
        launch_s = ev.ms * 1e-3 / steps
        rounds = max(2, -(-steps // n_sets))
        for i in range(n_sets):
            step(i)
        at.synchronize()
        with at.hip_event_timer() as ev:
            for _ in range(rounds):
                for i in range(n_sets):
                    step(i)
        cold_s = ev.ms * 1e-3 / (rounds * n_sets)
        results.append({"kernel": kernel, "inputs": [list(s) for s in in_shapes], "launch_us": launch_s * 1e6,
                        "algorithmic_bytes": abytes, "frac": abytes / launch_s * 1e-9 / HBM_PEAK_GBS,
                        "buffer_sets": n_sets, "launch_us_cold": cold_s * 1e6,
                        "frac_cold": abytes / cold_s * 1e-9 / HBM_PEAK_GBS,
                        "schedule": schedule_line(engine.GetLastImplementation())})
        results[-1]["functions"], results[-1]["kernel_source_sha1_16"] = kernel_identity(engine)
        flops = flops_as_written(kernel, in_shapes, out_shape)
        if flops:
            # a contraction: its arithmetic against the FP64 peak (vector and matrix peaks are equal) beside its bytes
            # against HBM; the larger of the two fractions is the one of the roofline that bounds the kernel
            results[-1]["tflops_cold"] = flops / cold_s * 1e-12
            results[-1]["frac_fp64_cold"] = flops / cold_s * 1e-9 / FP64_PEAK_GFLOPS
            # (which roof bounds it is a property of the kernel, not of the measurement: arithmetic per byte against the
            # machine balance of 78.6 TFLOP/s over 8 TB/s = 9.8)
            results[-1]["bound"] = "mfma" if flops / abytes > FP64_PEAK_GFLOPS / HBM_PEAK_GBS else "hbm"
        del sets, tensors
    # kernels bound by arithmetic (a large matrix product) are priced against the FP64 peak and kept out of the HBM means
    streaming = [r for r in results if r.get("bound") != "mfma"]
    mean = math.exp(sum(math.log(r["frac"]) for r in streaming) / len(streaming))
    mean_cold = math.exp(sum(math.log(r["frac_cold"]) for r in streaming) / len(streaming))
    total_s = sum(r["launch_us_cold"] for r in results) * 1e-6
    own = [r["frac_fp64_cold"] if r.get("bound") == "mfma" else r["frac_cold"] for r in results]
    mean_roofline = math.exp(sum(math.log(f) for f in own) / len(own))
    return {
        "metric": "fraction of the HBM peak, geometric mean over the %d of %d single-kernel shapes that HBM bounds, buffers rotated (1 GPU)" % (len(streaming), len(results)),
        "value": mean_cold, "value_warm": mean, "value_of_each_kernels_own_roofline": mean_roofline,
        "unit": "fraction of 8 TB/s", "n_gpus": 1, "steps": steps, "warmup": 5,
        "ms_per_step": total_s * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f64",
        "data": "synthetic", "config": {"workload": "kernel shapes, one launch each per step"},
        "seconds": time.perf_counter() - t_start, "kernels": results,
    }


def next_rows(at, workloads, args):
    """The steps either side of the operator apply at the size of the headline mesh: node vector <-> element vector,
    geometric-factor setup from the Jacobians, and scatter + apply in one launch; each with its launch time by HIP
    events on one buffer set and rotated, the kernel it ran, and the compiled reference on one host core."""
    import numpy as np
    block = {}
    for name in ("scatter", "sumgather", "jdsetup", "scatter_apply"):
        engine, steps_list, label, units, unit_name, abytes, flops = build_sets(at, workloads, name, args.rotate)
        wall, launch_s, roofline = measure_case(at, engine, steps_list, abytes, flops, 100, 10, args.settle_seconds,
                                                PRECOMPILED.get(name))
        block[name] = {
            "workload": label, "launch_us": launch_s * 1e6, "algorithmic_bytes": abytes, "frac": roofline["frac"],
            "buffer_sets": roofline["buffer_sets"], "launch_us_cold": roofline["launch_us_cold"],
            "frac_cold": roofline["frac_cold"], "value_cold": units / (roofline["launch_us_cold"] * 1e-6) * 1e-9,
            "unit": unit_name, "traffic": roofline["traffic"], "kernel": roofline["kernel"],
            "kernel_source_sha1_16": roofline["kernel_source_sha1_16"],
        }
        del engine, steps_list
        if args.no_cpu_baseline:
            continue
        checker, kind = host_checker()
        dofs, nodes = memo(workloads.hex_mesh_dof_map, 64, 64, 64, 3)
        if name in ("scatter", "sumgather"):
            L = memo(workloads.counter_uniform, 0xAC26, 0, (nodes,), -1.0, 1.0)
            Ev = memo(workloads.counter_uniform, 0xAC26, 1, (dofs.size,), -1.0, 1.0)
            flat = dofs.ravel()
            passes = 3
            t0 = time.perf_counter()
            for _ in range(passes):
                if name == "scatter":
                    checker.scatter(L, flat)
                else:
                    checker.sum_gather(Ev, flat, nodes)
            dt = (time.perf_counter() - t0) / passes
            value, sample = dofs.size / dt * 1e-9, "whole mesh, mean of %d passes of %.3f s" % (passes, dt)
        elif name == "jdsetup":
            n, Q = 2048, 10
            J = 0.1 * memo(workloads.counter_uniform, 0xAC28, 2, (n, Q, Q, Q, 3, 3), -1.0, 1.0) + np.eye(3)
            W = memo(workloads.counter_uniform, 0xAC28, 0, (Q, Q, Q), 0.1, 1.0)
            C = memo(workloads.counter_uniform, 0xAC28, 1, (n, Q, Q, Q), 0.5, 1.5)
            D = np.zeros((n, 3, 3, Q, Q, Q))
            t0 = time.perf_counter()
            Jinv, Jdet = checker.batch_matrix_inv_det(J)
            checker.contract("D_e_m_n_k1_k2_k3 = W_k1_k2_k3 C_e_k1_k2_k3 Jdet_e_k1_k2_k3 Jinv_e_k1_k2_k3_n_j Jinv_e_k1_k2_k3_m_j",
                             D, W, C, Jdet, Jinv, Jinv)
            dt = time.perf_counter() - t0
            value, sample = n * Q ** 3 / dt * 1e-9, "%d of 16384 elements, inverse + determinant + contraction, one pass, %.1f s" % (n, dt)
        else:
            n = 65536
            wl = workloads.config4(E=n)
            L = memo(workloads.counter_uniform, 0xAC29, 0, (nodes,), -1.0, 1.0)
            t0 = time.perf_counter()
            wl.arrays["X"] = checker.scatter(L, dofs[:n].ravel()).reshape(n, 4, 4, 4)
            workloads.run_on_checker(wl, checker)
            dt = time.perf_counter() - t0
            value, sample = wl.dof / dt * 1e-9, "%d of 262144 elements, scatter + 7-kernel chain, one pass, %.1f s" % (n, dt)
        block[name]["cpu_baseline"] = {"value": value, "unit": unit_name, "cores": 1, "kind": kind, "sample": sample}
    return block


def build_case(at, workloads, name, engine=None):
    """Tensors on the device and a step function for one workload: cfg1 / cfg2 / cfg3 / cfg5 at the sizes of the
    baseline configurations, FlatIndexedScatter / FlatIndexedSumGather on the headline mesh, and the other pipelines.
    Every call allocates a buffer set of its own (same values); calls that pass the same engine share its kernels.
    Returns (engine, step, label, units per step, unit name, algorithmic bytes, flops as written)."""
    if engine is None:
        engine = at.TensorEngine("HIP")
    if name == "cfg2":
        J = memo(workloads.config2_inputs)
        E, Q = J.shape[:2]
        tJ, Jinv, Jdet = at.Tensor(*J.shape), at.Tensor(*J.shape), at.Tensor(E, Q)
        tJ.data[...] = J
        for t in (tJ, Jinv, Jdet):
            t.MoveToGPU()
        step = lambda: engine.BatchMatrixInvDet(Jinv, Jdet, tJ)
        label = "configs[1]: BatchMatrixInvDet, J[65536,64,3,3]"
        units, unit_name, abytes, flops = E * Q, "Gmatrices/s", E * Q * 152, E * Q * 54
    elif name == "dsetup":
        # geometric factors of the diffusion operator from the inverse Jacobians (reference
        # unittest/kernel/test_TensorEngine.cpp:543-590), at the quadrature size of configs[4], E = 16384
        import numpy as np
        E, Q = 16384, 10
        W, C, Jdet = at.Tensor(Q, Q, Q), at.Tensor(E, Q, Q, Q), at.Tensor(E, Q, Q, Q)
        Jinv, D = at.Tensor(E, Q, Q, Q, 3, 3), at.Tensor(E, 3, 3, Q, Q, Q)
        W.data[...] = memo(workloads.counter_uniform, 0xAC27, 0, (Q, Q, Q), 0.1, 1.0)
        C.data[...] = memo(workloads.counter_uniform, 0xAC27, 1, (E, Q, Q, Q), 0.5, 1.5)
        Jdet.data[...] = memo(workloads.counter_uniform, 0xAC27, 2, (E, Q, Q, Q), 0.5, 1.5)
        Jinv.data[...] = memo(workloads.counter_uniform, 0xAC27, 3, (E, Q, Q, Q, 3, 3), -1.0, 1.0)
        for t in (W, C, Jdet, Jinv, D):
            t.MoveToGPU()
        k = "D_e_m_n_k1_k2_k3 = W_k1_k2_k3 C_e_k1_k2_k3 Jdet_e_k1_k2_k3 Jinv_e_k1_k2_k3_n_j Jinv_e_k1_k2_k3_m_j"
        step = lambda: engine(k, D, W, C, Jdet, Jinv, Jinv)
        label = "geometric factor setup D[16384,3,3,10,10,10] from Jinv, Jdet, C, W"
        points = E * Q * Q * Q
        abytes, flops = points * (9 + 1 + 1 + 9) * 8, points * 9 * 3 * 5
        units, unit_name = points, "Gpoints/s"
    elif name == "jdsetup":
        # the same geometric factors straight from the Jacobians: inverse, determinant and the contraction recorded as
        # one launch, Jinv and Jdet transient (they never reach device memory)
        E, Q = 16384, 10
        W, C, J = at.Tensor(Q, Q, Q), at.Tensor(E, Q, Q, Q), at.Tensor(E, Q, Q, Q, 3, 3)
        Jinv, Jdet, D = at.Tensor(E, Q, Q, Q, 3, 3), at.Tensor(E, Q, Q, Q), at.Tensor(E, 3, 3, Q, Q, Q)
        W.data[...] = memo(workloads.counter_uniform, 0xAC28, 0, (Q, Q, Q), 0.1, 1.0)
        C.data[...] = memo(workloads.counter_uniform, 0xAC28, 1, (E, Q, Q, Q), 0.5, 1.5)
        J.data[...] = memo(workloads.counter_uniform, 0xAC28, 2, (E, Q, Q, Q, 3, 3), -0.1, 0.1)
        J.data[...] += [[1.0, 0.0, 0.0], [0.0, 1.0, 0.0], [0.0, 0.0, 1.0]]
        for t in (Jinv, Jdet):
            t.SetTransient(True)
        for t in (W, C, J, Jinv, Jdet, D):
            t.MoveToGPU()
        k = "D_e_m_n_k1_k2_k3 = W_k1_k2_k3 C_e_k1_k2_k3 Jdet_e_k1_k2_k3 Jinv_e_k1_k2_k3_n_j Jinv_e_k1_k2_k3_m_j"

        def step():
            engine.BeginMultiKernelLaunch()
            engine.BatchMatrixInvDet(Jinv, Jdet, J)
            engine(k, D, W, C, Jdet, Jinv, Jinv)
            engine.EndMultiKernelLaunch()
        label = "geometric factor setup D[16384,3,3,10,10,10] from J, C, W in one launch (inverse and determinant in registers)"
        points = E * Q * Q * Q
        abytes, flops = points * (9 + 1 + 9) * 8, points * (9 * 3 * 5 + 54)
        units, unit_name = points, "Gpoints/s"
    elif name in ("scatter_apply", "scatter_then_apply"):
        # node vector -> element vector -> p=3 mass apply on the headline mesh (64^3 elements).  scatter_apply records
        # the scatter in the multi-kernel launch with a transient element vector, so the chain reads the node vector
        # through the element-to-node map and the element vector never exists; scatter_then_apply runs the two steps
        # one after the other.
        import numpy as np
        wl = memo(workloads.config4, 262144)
        tensors = workloads.bind_to_engine(wl, at, transient=True)
        dofs, nodes = memo(workloads.hex_mesh_dof_map, 64, 64, 64, 3)
        M = at.IndexMapping(nodes, dofs.size)
        M.map[:] = dofs.ravel()
        L = at.Tensor(nodes)
        L.data[...] = memo(workloads.counter_uniform, 0xAC29, 0, (nodes,), -1.0, 1.0)
        tensors["X"].SetTransient(name == "scatter_apply")
        for t in list(tensors.values()) + [L]:
            t.MoveToGPU()
        engine.FlatIndexedScatter(tensors["X"], L, M)        # moves the map to the device

        def step():
            if name == "scatter_apply":
                engine.BeginMultiKernelLaunch()
                engine.FlatIndexedScatter(tensors["X"], L, M)
            else:
                engine.FlatIndexedScatter(tensors["X"], L, M)
                engine.BeginMultiKernelLaunch()
            for k, out, ins in wl.kernels:
                engine(k, tensors[out], *[tensors[i] for i in ins])
            engine.EndMultiKernelLaunch()
        label = ("node vector [7189057] -> p=3 mass apply on 262144 elements, " +
                 ("element vector read through the map in one launch" if name == "scatter_apply"
                  else "scatter and apply as two steps"))
        E = 262144
        abytes = dofs.size * 4 + nodes * 8 + E * (1000 + 512)
        if name == "scatter_then_apply":
            abytes += 2 * dofs.size * 8                      # the element vector written, then read
        flops = wl.flops
        units, unit_name = wl.dof, "GDOF/s"
    elif name == "operator":
        # one dense 64 x 64 operator applied to 2^18 vectors: the one GEMM-shaped kernel of this engine (FP64 matrix cores)
        E, n = 1 << 18, 64
        B, X, A = at.Tensor(n, n), at.Tensor(E, n), at.Tensor(E, n)
        B.data[...] = memo(workloads.counter_uniform, 0xAC28, 0, (n, n), -1.0, 1.0)
        X.data[...] = memo(workloads.counter_uniform, 0xAC28, 1, (E, n), -1.0, 1.0)
        for t in (B, X, A):
            t.MoveToGPU()
        step = lambda: engine("A_e_i = B_i_j X_e_j", A, B, X)
        label = "A[262144,64] = B[64,64] X[262144,64], one dense operator applied to every vector"
        abytes, flops = (2 * E * n + n * n) * 8, 2 * E * n * n
        units, unit_name = E * n, "GDOF/s"
    elif name == "dense_apply":
        # a dense element operator applied, weighted at the quadrature points and applied back: 27 dofs (p=2 hex),
        # 64 points, both products in one matrix-core kernel, the intermediate transient
        E, nd, nq = 1 << 19, 27, 64
        B, X, D, U, Y = at.Tensor(nq, nd), at.Tensor(E, nd), at.Tensor(E, nq), at.Tensor(E, nq), at.Tensor(E, nd)
        B.data[...] = memo(workloads.counter_uniform, 0xAC29, 0, (nq, nd), -1.0, 1.0)
        X.data[...] = memo(workloads.counter_uniform, 0xAC29, 1, (E, nd), -1.0, 1.0)
        D.data[...] = memo(workloads.counter_uniform, 0xAC29, 2, (E, nq), 0.5, 1.5)
        U.SetTransient(True)
        for t in (B, X, D, U, Y):
            t.MoveToGPU()

        def step():
            engine.BeginMultiKernelLaunch()
            engine("U_e_k = B_k_j X_e_j D_e_k", U, B, X, D)
            engine("Y_e_i = B_k_i U_e_k", Y, B, U)
            engine.EndMultiKernelLaunch()
        label = "Y[524288,27] = Bt (D o (B X)), B[64,27], D[524288,64]: dense element operator in one launch"
        abytes, flops = (E * (nd + nq + nd) + nq * nd) * 8, E * (4 * nq * nd + nq)
        units, unit_name = E * nd, "GDOF/s"
    elif name in ("matmul", "matmul_batched"):
        # a plain matrix product, the kernel of the reference's first test (unittest/kernel/test_TensorEngine.cpp:47-77,
        # "A_i_j = B_i_k C_k_j") at 4 096 x 4 096, and products of 128 x 128 element matrices: tiled product schedule
        # on the FP64 matrix cores; the first is bound by arithmetic
        import numpy as np
        if name == "matmul":
            n = 4096
            shapes, k = [(n, n)] * 3, "A_i_j = B_i_k C_k_j"
            label, flops, units, unit_name = "A[4096,4096] = B[4096,4096] C[4096,4096]", 2 * n ** 3, n * n, "Gentries/s"
        else:
            E, n = 1024, 128
            shapes, k = [(E, n, n)] * 3, "A_e_i_j = B_e_i_k C_e_k_j"
            label, flops, units, unit_name = "A[1024,128,128] = B[1024,128,128] C[1024,128,128] per entry", 2 * E * n ** 3, E * n * n, "Gentries/s"
        A, B, C = (at.Tensor(*shp) for shp in shapes)
        B.data[...] = memo(workloads.counter_uniform, 0xAC2B, 0, shapes[1], -1.0, 1.0)
        C.data[...] = memo(workloads.counter_uniform, 0xAC2B, 1, shapes[2], -1.0, 1.0)
        for t in (A, B, C):
            t.MoveToGPU()
        step = lambda: engine(k, A, B, C)
        abytes = 3 * 8 * int(np.prod(shapes[0]))
    elif name == "stiffness":
        # 3D stiffness matrix assembly, the 12-loop kernel of the reference's tests
        # (unittest/kernel/test_TensorEngine.cpp:437-496) at 8 192 elements: 1 125 terms of 4 factors per output as
        # written; `flops` counts the arithmetic of the two steps it is evaluated as (k3 first, then 225 terms per
        # output: one product shared by a 5 x 5 tile of outputs and one multiply-add per output)
        E = 8192
        S, D = at.Tensor(E, 5, 5, 5, 5, 5, 5), at.Tensor(E, 5, 5, 5, 3, 3)
        tables = [at.Tensor(5, 5, 5, 3, 3) for _ in range(3)]
        for i, t in enumerate(tables):
            t.data[...] = memo(workloads.counter_uniform, 0xAC2A, i, (5, 5, 5, 3, 3), -1.0, 1.0)
        D.data[...] = memo(workloads.counter_uniform, 0xAC2A, 3, (E, 5, 5, 5, 3, 3), 0.5, 1.5)
        for t in tables + [S, D]:
            t.MoveToGPU()
        k = "S_e_i1_i2_i3_j1_j2_j3 = B1_i1_j1_k1_m_n B2_i2_j2_k2_m_n B3_i3_j3_k3_m_n D_e_k1_k2_k3_m_n"
        step = lambda: engine(k, S, tables[0], tables[1], tables[2], D)
        label = "3D stiffness assembly S[8192,5,5,5,5,5,5] from three tables [5,5,5,3,3] and D[8192,5,5,5,3,3]"
        abytes = (E * (15625 + 1125) + 3 * 1125) * 8
        flops = E * (5625 * 5 * 2 + 625 * 225 * (1 + 2 * 25))
        units, unit_name = E * 15625, "Gentries/s"
    elif name in ("scatter", "sumgather"):
        # node vector <-> element vector of the headline mesh size: 64^3 hex elements of degree 3
        import numpy as np
        dofs, nodes = memo(workloads.hex_mesh_dof_map, 64, 64, 64, 3)
        M = at.IndexMapping(nodes, dofs.size)
        M.map[:] = dofs.ravel()
        L, Ev = at.Tensor(nodes), at.Tensor(dofs.size)
        L.data[...] = memo(workloads.counter_uniform, 0xAC26, 0, (nodes,), -1.0, 1.0)
        Ev.data[...] = memo(workloads.counter_uniform, 0xAC26, 1, (dofs.size,), -1.0, 1.0)
        for t in (L, Ev):
            t.MoveToGPU()
        if name == "scatter":
            step = lambda: engine.FlatIndexedScatter(Ev, L, M)
            label = "E-vector[262144*64] = L-vector[7189057] through the element-to-node map"
            abytes = dofs.size * (4 + 8) + nodes * 8          # map + E-vector written + every node read once
        else:
            step = lambda: engine.FlatIndexedSumGather(L, Ev, M)
            label = "L-vector[7189057] = sum of E-vector[262144*64] entries through the element-to-node map"
            abytes = dofs.size * (4 + 8) + nodes * (4 + 8)    # inverse map + E-vector read + row offsets + L written
        units, unit_name, flops = dofs.size, "GDOF/s", dofs.size
    elif name == "cfg5":
        # inputs for 2048 elements, repeated 32 times along the element index on the device (generating and
        # uploading all 4.7 GB of geometric factors from the host takes minutes; no timing depends on the values)
        period, times = 2048, 32
        small = memo(workloads.config5, period)
        tensors = workloads.bind_to_engine_repeated(small, at, engine, times, transient=True)
        wl = small
        step = lambda: workloads.launch(wl, engine, tensors)
        label = ("configs[4]: p=7 hex diffusion apply, E=65536, 18-kernel multi-kernel launch, intermediates transient "
                 "(input values repeat with a period of %d elements)" % period)
        abytes, flops = small.algorithmic_bytes * times, small.flops * times
        units, unit_name = small.dof * times, "GDOF/s"
    else:
        wl = memo({"cfg1": workloads.config1, "cfg3": workloads.config3}[name])
        tensors = workloads.bind_to_engine(wl, at, transient=True, inputs_only=True)
        for t in tensors.values():
            t.MoveToGPU()
        step = lambda: workloads.launch(wl, engine, tensors)
        label = {"cfg1": "configs[0]: S_i_j = A_n_i_j B_n, n=2^20", "cfg3": "configs[2]: p=2 hex mass assembly, E=32768"}[name]
        abytes, flops = wl.algorithmic_bytes, wl.flops
        units, unit_name = abytes, "GB/s"
    return engine, step, label, units, unit_name, abytes, flops


PRECOMPILED = {"cfg2": "batchMatrixKernel<3,inv,det>", "scatter": "scatterKernel2", "sumgather": "sumGatherKernel"}


def build_sets(at, workloads, name, rotate=0):
    """One buffer set to time re-launches on (the first) plus as many more as it takes to push a set out of the
    memory-side cache between two launches on it.  Returns (engine, [step per set], label, units, unit name,
    algorithmic bytes, flops)."""
    engine, step, label, units, unit_name, abytes, flops = build_case(at, workloads, name)
    steps = [step]
    for _ in range(sets_beyond_the_last_level_cache(abytes, rotate) - 1):
        steps.append(build_case(at, workloads, name, engine)[1])
    return engine, steps, label, units, unit_name, abytes, flops


def measure_case(at, engine, steps_list, abytes, flops, steps, warmup, settle_seconds, precompiled=None):
    """Times one workload twice with HIP events: re-launched on one buffer set (`launch_us`, `frac`: whatever of the
    set fits the 256 MB memory-side cache is served from there), and launched round-robin over all the sets
    (`launch_us_cold`, `frac_cold`: every byte comes from and goes to HBM).  With one set the two are the same
    measurement."""
    if callable(steps_list):
        steps_list = [steps_list]
    step = steps_list[0]
    if ONLY_ROTATED and len(steps_list) > 1:
        # every launch of the run, settling and warm-up included, goes round-robin over the buffer sets (for kernel
        # traces, whose per-kernel averages then are those of launches on data that comes from HBM)
        turn = [0]

        def step():
            turn[0] += 1
            steps_list[turn[0] % len(steps_list)]()
    # sustained load before anything is timed (see settle_clocks): bursts of launches, not one launch per
    # synchronisation, or the device drops back to idle clocks between them
    for s in steps_list:
        s()
    at.synchronize()
    t0 = time.perf_counter()
    step()
    at.synchronize()
    burst = max(1, min(100, int(2e-3 / max(time.perf_counter() - t0, 1e-6))))
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < settle_seconds:
        for _ in range(burst):
            step()
        at.synchronize()
    for _ in range(warmup):
        step()
    at.synchronize()
    t0 = time.perf_counter()
    with at.hip_event_timer() as ev:
        for _ in range(steps):
            step()
    at.synchronize()
    wall = time.perf_counter() - t0
    launch_s = ev.ms * 1e-3 / steps
    achieved = abytes / launch_s * 1e-9
    names, digest = kernel_identity(engine, precompiled)
    roofline = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": achieved / HBM_PEAK_GBS, "traffic": measured_traffic(engine, precompiled), "algorithmic_bytes": abytes,
                "launch_us": launch_s * 1e6, "kernel": names[0] if names else None, "kernel_source_sha1_16": digest}
    cold_s = launch_s
    n = len(steps_list)
    if n > 1:
        rounds = max(2, -(-steps // n))
        for _ in range(max(1, warmup // n)):
            for s in steps_list:
                s()
        at.synchronize()
        with at.hip_event_timer() as ev:
            for _ in range(rounds):
                for s in steps_list:
                    s()
        at.synchronize()
        cold_s = ev.ms * 1e-3 / (rounds * n)
    roofline.update({"buffer_sets": n, "launch_us_cold": cold_s * 1e6, "achieved_cold": abytes / cold_s * 1e-9,
                     "frac_cold": abytes / cold_s * 1e-9 / HBM_PEAK_GBS})
    return wall, launch_s, roofline


def all_configs(at, workloads, args):
    """cfg1 / cfg2 / cfg3 / cfg5 at their full sizes, one after the other: GPU figures by HIP events and the host
    baseline beside each."""
    block = {}
    for name in ("cfg1", "cfg2", "cfg3", "cfg5"):
        engine, steps_list, label, units, unit_name, abytes, flops = build_sets(at, workloads, name, args.rotate)
        steps = 50 if name == "cfg5" else 200
        wall, launch_s, roofline = measure_case(at, engine, steps_list, abytes, flops, steps, 10, args.settle_seconds,
                                                PRECOMPILED.get(name))
        block[name] = {
            "workload": label, "launch_us": launch_s * 1e6, "steps": steps, "algorithmic_bytes": abytes,
            "GBps": roofline["achieved"], "frac": roofline["frac"], "gflops_as_written": flops / launch_s * 1e-9,
            "value": units / launch_s * 1e-9, "unit": unit_name, "buffer_sets": roofline["buffer_sets"],
            "launch_us_cold": roofline["launch_us_cold"], "GBps_cold": roofline["achieved_cold"],
            "frac_cold": roofline["frac_cold"], "traffic": roofline["traffic"],
            "kernel": roofline["kernel"], "kernel_source_sha1_16": roofline["kernel_source_sha1_16"],
        }
        if name == "cfg1":
            block[name]["graph_replay_us"] = graph_replay_us(at, steps_list[0], 500)
        del engine, steps_list
        if not args.no_cpu_baseline:
            block[name]["cpu_baseline"] = cpu_baseline_for(name, workloads)
    return block


def graph_replay_us(at, step, replays):
    """The step recorded once as a launch sequence (hipGraph) and replayed: time per replay by HIP events."""
    step()
    at.synchronize()
    with at.recorded_launches() as seq:
        step()
    for _ in range(50):
        seq.launch()
    at.synchronize()
    with at.hip_event_timer() as ev:
        for _ in range(replays):
            seq.launch()
    at.synchronize()
    return ev.ms * 1e3 / replays


def cfg1_sizes(at, args):
    """The batched reduction of configs[0] at other lengths n: per-step time by HIP events (both launches of the
    split contraction), algorithmic GB/s, and what is left over the time the bytes need at 6.5 TB/s (the rate the
    same kernel reaches at n = 2^24).  At n = 2048 the bytes are negligible: that row is the cost of the two dependent
    launches alone."""
    engine = at.TensorEngine("HIP")
    rows = []
    for n in (2048, 16384, 65536, 262144, 524288, 1 << 20, 1 << 21, 1 << 22, 1 << 24):
        A, B, S = at.Tensor(n, 3, 3), at.Tensor(n), at.Tensor(3, 3)
        for t in (A, B, S):
            t.SwitchToGPU()
            t.Set(1.0)
        step = lambda: engine("S_i_j = A_n_i_j B_n", S, A, B)
        for _ in range(50):
            step()
        at.synchronize()
        steps = 500 if n <= (1 << 21) else 100
        with at.hip_event_timer() as ev:
            for _ in range(steps):
                step()
        us = ev.ms * 1e3 / steps
        nbytes = (n * 10 + 9) * 8
        rows.append({"n": n, "us_per_step": us, "GBps": nbytes / us * 1e-3, "frac": nbytes / us * 1e-3 / HBM_PEAK_GBS,
                     "us_of_bytes_at_6500_GBps": nbytes / 6.5e6, "us_beyond_that": us - nbytes / 6.5e6})
        del A, B, S
    at_full = [r for r in rows if r["n"] == 1 << 20][0]
    return {"metric": "cfg1 batched reduction at other lengths (1 GPU)", "value": at_full["GBps"], "unit": "GB/s", "n_gpus": 1,
            "steps": 500, "warmup": 50, "ms_per_step": at_full["us_per_step"] * 1e-3, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "f64", "data": "synthetic",
            "config": {"workload": "S_i_j = A_n_i_j B_n for n = 2^11 .. 2^24; value is the n = 2^20 row"}, "sizes": rows}


def other_workload(at, workloads, args):
    name = args.workload
    engine, steps_list, label, units, unit_name, abytes, flops = build_sets(at, workloads, name, args.rotate)
    steps, warmup = min(args.steps, 200), min(args.warmup, 20)
    wall, launch_s, roofline = measure_case(at, engine, steps_list, abytes, flops, steps, warmup, args.settle_seconds,
                                            PRECOMPILED.get(name))
    result = {
        "metric": "%s throughput (1 GPU)" % name, "value": units * steps / wall * 1e-9, "unit": unit_name, "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": wall / steps * 1e3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f64", "data": "synthetic", "config": {"workload": label},
        "gflops_as_written": flops / launch_s * 1e-9, "roofline": roofline,
    }
    if name == "stiffness":
        # this one is bound by arithmetic, not by memory: say so beside the HBM figures
        result["gflops_as_evaluated"] = result.pop("gflops_as_written")
        result["fp64_vector_peak_frac"] = flops / launch_s * 1e-9 / FP64_PEAK_GFLOPS
    if name in ("matmul", "matmul_batched"):
        # the roofline that bounds a large matrix product is the FP64 matrix peak (78.6 TFLOP/s), not HBM
        result["hbm"] = {k: roofline[k] for k in ("achieved", "frac", "achieved_cold", "frac_cold") if k in roofline}
        cold_s = roofline.get("launch_us_cold", launch_s * 1e6) * 1e-6
        fp64 = {"bound": "mfma", "achieved": flops / launch_s * 1e-12, "peak": FP64_PEAK_GFLOPS * 1e-3, "unit": "TFLOP/s",
                "frac": flops / launch_s * 1e-9 / FP64_PEAK_GFLOPS, "achieved_cold": flops / cold_s * 1e-12,
                "frac_cold": flops / cold_s * 1e-9 / FP64_PEAK_GFLOPS, "traffic": None}
        for key in ("launch_us", "launch_us_cold", "buffer_sets", "kernel", "kernel_source_sha1_16", "algorithmic_bytes"):
            if key in roofline:
                fp64[key] = roofline[key]
        if name == "matmul" or fp64["frac_cold"] > roofline.get("frac_cold", 0.0):
            result["roofline"] = fp64
        else:
            result["fp64_matrix_peak"] = fp64
    if name in ("cfg1", "cfg2", "cfg3", "cfg5") and not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline_for(name, workloads)
    return result


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--settle-seconds", type=float, default=0.25,
                    help="untimed launches before the warm-up, until clocks have settled under sustained load")
    ap.add_argument("--rotate", type=int, default=0,
                    help="buffer sets that the cold figures rotate over: 0 (default) as many as it takes to exceed 1 GiB "
                         "together, 1 none (cold figures then repeat the ordinary ones), N that many")
    ap.add_argument("--only-rotated", action="store_true",
                    help="every launch of the run (settling, warm-up, timed) goes round-robin over the buffer sets, so a "
                         "kernel trace of the run averages launches on data from HBM only; the same-buffer figures of "
                         "the line then repeat the rotated ones")
    ap.add_argument("--elements", type=int, default=262144)
    ap.add_argument("--cpu-sample-elems", type=int, default=262144)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-store-all", action="store_true")
    ap.add_argument("--no-all-configs", action="store_true",
                    help="leave out the block with the other four baseline configurations")
    ap.add_argument("--no-next-rows", action="store_true",
                    help="leave out the block with scatter, sum-gather, geometric-factor setup and scatter + apply")
    ap.add_argument("--no-shapes", action="store_true", help="leave out the summary of the single-kernel shapes")
    ap.add_argument("--workload", default="cfg4", choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg5", "scatter", "sumgather", "dsetup", "jdsetup", "scatter_apply", "scatter_then_apply", "operator", "dense_apply", "stiffness", "matmul", "matmul_batched", "shapes", "cfg1_sizes"],
                    help="cfg4 (default) is the headline metric; the others print the same kind of line for the "
                         "remaining baseline configurations at their full sizes and for the node-vector <-> "
                         "element-vector steps either side of the operator apply")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one scale-by-1.0 kernel over X (reads and writes E*512 bytes): the known-size "
                         "kernel that hardware-counter runs are scaled by")
    args = ap.parse_args()
    global ONLY_ROTATED
    ONLY_ROTATED = args.only_rotated
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (the workload shards over elements "
                 "without any exchange, so N GPUs would each run this same kernel on 1/N of them).  Run with --gpus 1.")

    import acrotensor_amd as at
    from acrotensor_amd import workloads

    if not at.is_hip_ready():
        sys.exit("bench.py needs a HIP device; there is no host fallback.")

    if args.workload == "shapes":
        print(json.dumps(kernel_shapes(at, args)))
        return
    if args.workload == "cfg1_sizes":
        print(json.dumps(cfg1_sizes(at, args)))
        return
    if args.workload != "cfg4":
        print(json.dumps(other_workload(at, workloads, args)))
        return

    wl = workloads.config4(E=args.elements)
    engine = at.TensorEngine("HIP")
    n_sets = sets_beyond_the_last_level_cache(wl.algorithmic_bytes, args.rotate)
    sets = []
    for _ in range(n_sets):
        bound = workloads.bind_to_engine(wl, at, transient=True, inputs_only=True)
        for name, t in bound.items():
            if name in wl.inputs:
                t.MoveToGPU()
            else:
                t.SwitchToGPU()                              # written before it is read: device memory only
        sets.append(bound)
    tensors = sets[0]

    if args.calibration_copy:
        tensors["X"].Mult(1.0)
        at.synchronize()

    if ONLY_ROTATED:
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < args.settle_seconds:
            time_steps_rotating(at, workloads, wl, engine, sets, 100, 0)
        wall, dev = time_steps_rotating(at, workloads, wl, engine, sets, args.steps, args.warmup)
    else:
        settle_clocks(at, workloads, wl, engine, tensors, args.settle_seconds)
        wall, dev = time_steps(at, workloads, wl, engine, tensors, args.steps, args.warmup)
    ms_per_step = wall / args.steps * 1e3
    launch_s = dev / args.steps
    achieved = wl.algorithmic_bytes / launch_s * 1e-9
    # the same steps round-robin over the buffer sets: no byte of a set survives in the memory-side cache until
    # the set's next launch
    wall_cold, dev_cold = time_steps_rotating(at, workloads, wl, engine, sets, args.steps, args.warmup)
    cold_s = dev_cold / args.steps
    achieved_cold = wl.algorithmic_bytes / cold_s * 1e-9

    result = {
        "metric": METRIC,
        "value": wl.dof * args.steps / wall * 1e-9,
        "unit": "GDOF/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f64",
        "data": "synthetic",
        "config": {
            "workload": "configs[3]: p=3 sum-factorised hex mass apply, E=%d, B[5,4] X[E,4,4,4] D[E,5,5,5], "
                        "7-kernel multi-kernel launch, intermediates T1..V2 marked transient" % args.elements,
            "elements": args.elements,
            "dof": wl.dof,
            "seed": wl.seed,
        },
        "pct_hbm_peak": 100.0 * achieved / HBM_PEAK_GBS,
        "kernel_gdof_per_s": wl.dof / launch_s * 1e-9,
        "value_cold": wl.dof * args.steps / wall_cold * 1e-9,
        "pct_hbm_peak_cold": 100.0 * achieved_cold / HBM_PEAK_GBS,
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": measured_traffic(engine),
            "algorithmic_bytes": wl.algorithmic_bytes,
            "launch_us": launch_s * 1e6,
            "buffer_sets": n_sets,
            "launch_us_cold": cold_s * 1e6,
            "achieved_cold": achieved_cold,
            "frac_cold": achieved_cold / HBM_PEAK_GBS,
            "cold": "the same %d steps issued round-robin over %d sets of X, D and Y (distinct allocations, same "
                    "values, %.2f GB together): nothing a launch touches is left in the 256 MB memory-side cache "
                    "from the set's previous launch" % (args.steps, n_sets, n_sets * wl.algorithmic_bytes * 1e-9),
            "kernel": kernel_identity(engine)[0][0],
            "kernel_source_sha1_16": kernel_identity(engine)[1],
        },
    }

    if not args.no_store_all:
        for bound in sets:
            for name in wl.transient:
                bound[name].SetTransient(False)
        n2 = max(10, args.steps // 4)
        # The first launch compiles the other kernel while the device idles: settle again before timing.
        workloads.launch(wl, engine, tensors)
        at.synchronize()
        if ONLY_ROTATED:
            wall2, dev2 = time_steps_rotating(at, workloads, wl, engine, sets, n2, max(5, args.warmup // 4))
        else:
            settle_clocks(at, workloads, wl, engine, tensors, args.settle_seconds)
            wall2, dev2 = time_steps(at, workloads, wl, engine, tensors, n2, max(5, args.warmup // 4))
        wall2c, dev2c = time_steps_rotating(at, workloads, wl, engine, sets, n2, max(5, args.warmup // 4))
        stored_bytes = args.elements * (64 + 125 + 64 + 610) * 8
        moved = stored_bytes / (dev2 / n2) * 1e-9
        moved_cold = stored_bytes / (dev2c / n2) * 1e-9
        result["store_all"] = {
            "what": "the same launch with T1..V2 as ordinary tensors: every intermediate is also written to HBM, "
                    "as with the reference (what a caller gets who only changes the policy string)",
            "value": wl.dof * n2 / wall2 * 1e-9,
            "unit": "GDOF/s",
            "launch_us": dev2 / n2 * 1e6,
            "hbm_bytes_moved": stored_bytes,
            "achieved_GBs_incl_intermediates": moved,
            "frac_of_hbm_peak_on_bytes_moved": moved / HBM_PEAK_GBS,
            "launch_us_cold": dev2c / n2 * 1e6,
            "frac_of_hbm_peak_on_bytes_moved_cold": moved_cold / HBM_PEAK_GBS,
            "traffic": measured_traffic(engine),
            "kernel": kernel_identity(engine)[0][0],
            "kernel_source_sha1_16": kernel_identity(engine)[1],
        }
        for bound in sets:
            for name in wl.transient:
                bound[name].SetTransient(True)

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(workloads, min(args.cpu_sample_elems, args.elements))

    del tensors, sets, bound
    if not args.no_all_configs:
        result["all_configs"] = all_configs(at, workloads, args)
    if not args.no_next_rows:
        result["next_rows"] = next_rows(at, workloads, args)
    if not args.no_shapes:
        full = kernel_shapes(at, args)
        streaming = [r for r in full["kernels"] if r.get("bound") != "mfma"]
        worst = min(streaming, key=lambda r: r["frac_cold"])
        result["shapes_summary"] = {
            "what": "single kernels of other shapes (bench.py --workload shapes lists them): fraction of the HBM peak "
                    "by HIP events, buffers rotated, over the kernels that HBM bounds; those that arithmetic bounds "
                    "against the FP64 peak", "n": len(full["kernels"]), "n_hbm_bound": len(streaming),
            "geomean": full["value_warm"], "geomean_cold": full["value"], "min_cold": worst["frac_cold"],
            "min_cold_kernel": worst["kernel"], "min_cold_inputs": worst["inputs"],
            "bound_by_arithmetic": [{"kernel": r["kernel"], "inputs": r["inputs"], "tflops_cold": r["tflops_cold"],
                                     "frac_fp64_cold": r["frac_fp64_cold"]} for r in full["kernels"] if r.get("bound") == "mfma"],
            "geomean_of_each_kernels_own_roofline": full["value_of_each_kernels_own_roofline"], "seconds": full["seconds"]}

    print(json.dumps(result))


if __name__ == "__main__":
    main()
