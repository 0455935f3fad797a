#!/usr/bin/env python
"""Benchmark of the fused op-tree path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Headline (``value``): the fused Adam update of 25,000,000 fp32 parameters
(5000 x 5000) -- the three assigns of neon's Adam.optimize run as ONE kernel --
as whole-job GB/s over K steps: algorithmic bytes (4 tensors read + 3 written =
700 MB per step) divided by wall-clock time around the K ``be.begin / assigns /
be.end`` calls, inputs resident in HBM, stream synchronised on both sides.

``roofline`` is that kernel alone, timed with HIP events on the launch stream
around the same K launches.  ``per_config`` lists every benchmark op-tree
(elementwise + sigmoid, softmax, Adam fused and as three kernels, fp16 row
normalisation, argmax / max / cross-entropy over a 32000-row vocabulary) with
the same event timing, and cold-cache timings of those trees (launches
rotating over >= 768 MB of distinct tensors holding seeded random data).
Each row also carries ``kernel_us_rocprof`` -- the median rocprofv3 kernel
duration of the same kernel from the committed summaries under ``profiles/``
-- and ``traffic``, the HBM bytes per launch from hardware counters; both are
looked up by kernel name and are null when the summaries were made from
other kernels (the prebuilt kernels behind direct C-ABI entry points are found
by a part of the compiler's name for them, which a change of their source does
not alter: their rows are remade whenever ``kernels.hip`` changes).  ``cpu_baseline`` times the numpy oracle on the same Adam step
on this machine's host cores.

Other modes (each the program behind one of the summaries in ``profiles/``):
``--trace-pass hot|cold`` (rocprofv3 --kernel-trace), ``--counter-pass``
(rocprofv3 --pmc), ``--sweep DTYPE`` (wall clock over a grid of shapes),
``--configs-only`` / ``--no-cold`` (shorter tables).  The per-configuration
tables go to stderr after the JSON line, the benchmark configurations last.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# Figures that cannot be read from inside this process come from the committed rocprofv3 summaries (written by
# `python -m neon_amd.profile_summary` from profiled runs of `bench.py --counter-pass` / `--trace-pass`; each
# summary quotes its commands).  They are looked up by the NAME of the kernel that has just been timed here: when
# the generator has changed since a summary was made, the name differs and the figure is null, never stale.
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "hbm_traffic_all_configs_pmc.txt")
DURATION_SUMMARY = {"hot": os.path.join(ROOT, "profiles", "kernel_durations_hot_kernel_trace.txt"),
                    "cold": os.path.join(ROOT, "profiles", "kernel_durations_cold_kernel_trace.txt")}


def measured_traffic(kernel_name):
    """HBM bytes per launch of ``kernel_name`` (FETCH_SIZE + WRITE_SIZE, each scaled by a
    copy kernel of known size) from the committed counter summary, or None"""
    from neon_amd.profile_summary import lookup
    rec = lookup(TRAFFIC_SUMMARY, kernel_name)
    return rec["traffic_bytes"] if rec else None


def rocprof_us(kernel_name, mode="hot"):
    """median rocprofv3 kernel duration (>= 50 launches after >= 10 warm-ups) of
    ``kernel_name`` from the committed kernel-trace summary, or None"""
    from neon_amd.profile_summary import lookup
    rec = lookup(DURATION_SUMMARY[mode], kernel_name)
    return rec["median_us"] if rec else None


def rocprof_us_part(part, mode="hot"):
    """as ``rocprof_us`` for a prebuilt kernel, found by a part of the compiler's name for it"""
    from neon_amd.profile_summary import lookup_part
    rec = lookup_part(DURATION_SUMMARY[mode], part)
    return rec["median_us"] if rec else None


COLD_BYTES = 768 << 20         # tensor sets rotated through by the cold-cache rows


def _fresh(be, shape, dtype=np.float32, fill=None, rs=None, scale=1.0, shift=0.0):
    t = be.empty(shape, dtype=dtype)
    if rs is not None:
        # generate on the host in row blocks to bound host memory
        rows = shape[0]
        step = max(1, (1 << 24) // max(1, shape[1]))
        for r0 in range(0, rows, step):
            r1 = min(rows, r0 + step)
            blk = (rs.standard_normal((r1 - r0, shape[1])) * scale + shift).astype(np.float32).astype(dtype)
            t[r0:r1, :].set(blk) if (r0, r1) != (0, rows) else t.set(blk)
    elif fill is not None:
        t[:] = fill
    return t



class Case(object):
    """One benchmark op-tree: ``make(k)`` allocates the k-th set of its tensors
    (set 0 holds exactly the seeded inputs of ``neon_amd.configs``; the others
    the same values rolled by k, so that every set of a cold-cache rotation is
    random data too), ``issue(*tensors)`` states the tree."""

    def __init__(self, label, nbytes, elements, make, issue, cold=True, reps=50):
        self.label, self.nbytes, self.elements = label, nbytes, elements
        self.make, self.issue, self.cold, self.reps = make, issue, cold, reps

    def nsets(self):
        return max(3, min(600, -(-COLD_BYTES // self.nbytes)))


def baseline_cases(be):
    """the trees of the five benchmark configurations at their full shapes,
    plus the two floor kernels (the same structures on next to no data)"""
    from neon_amd import configs
    from neon_amd.backends.backend import Block
    f32, f16, i32 = np.float32, np.float16, np.int32
    roll = lambda a, k, axis=0: a if k == 0 else np.roll(a, 13 * k, axis=axis)
    cases = []
    host = {}

    def inputs(name):
        if name not in host:
            host[name] = getattr(configs, "inputs_" + name)()
        return host[name]

    n1 = configs.C1_SHAPE[0] * configs.C1_SHAPE[1]

    def make_c1(k):
        x, y = inputs("c1")
        return be.empty(configs.C1_SHAPE), be.array(roll(x, k)), be.array(roll(y, k))
    cases.append(Case("C1 fused sig(0.5x+2y) (4096,128) f32", configs.bytes_c1a(), n1, make_c1,
                      lambda o, x, y: configs.c1_fused(be, o, x, y)))
    cases.append(Case("C1a 0.5x+2y (4096,128) f32", configs.bytes_c1a(), n1, make_c1,
                      lambda o, x, y: configs.c1a(be, o, x, y)))

    def make_c1b(k):
        o = be.array(roll(inputs("c1")[0], k))
        return (o,)
    cases.append(Case("C1b sig in place (4096,128) f32", configs.bytes_c1b(), n1, make_c1b, lambda o: configs.c1b(be, o)))

    def make_c2(k):
        return be.empty(configs.C2_SHAPE), be.array(roll(inputs("c2")[0], k))
    cases.append(Case("C2 softmax axis0 (1000,128) f32", configs.bytes_c2(), configs.C2_SHAPE[0] * configs.C2_SHAPE[1],
                      make_c2, lambda o, x: configs.c2_softmax(be, o, x)))

    n3 = configs.C3_SHAPE[0] * configs.C3_SHAPE[1]
    step = [0]

    def make_c3(k):
        grad, param = inputs("c3")
        tensors = be.array(param), be.array(grad), be.zeros(configs.C3_SHAPE), be.zeros(configs.C3_SHAPE)
        host.pop("c3")
        return tensors

    def adam(p, g, m, v):
        step[0] += 1
        be.begin(Block.update, step[0])
        configs.c3_adam_step(be, p, g, m, v, step[0])
        be.end(Block.update, step[0])
    # (700 MB per launch: far beyond every cache, so one set is already a cold run)
    cases.append(Case("C3 Adam fused, 1 kernel (5000,5000) f32", configs.bytes_c3(fused=True), n3, make_c3, adam,
                      cold=False, reps=20))

    n4 = configs.C4_SHAPE[0] * configs.C4_SHAPE[1]
    shared = {}

    def make_c4(k):
        x, gamma, beta = inputs("c4")
        if "g4" not in shared:
            shared["g4"], shared["b4"] = be.array(gamma), be.array(beta)
        return (be.empty(configs.C4_SHAPE, dtype=f16), be.array(roll(x, k, axis=1), dtype=f16), shared["g4"], shared["b4"])
    cases.append(Case("C4 rownorm (256,100352) f16", configs.bytes_c4(), n4, make_c4,
                      lambda o, x, g, b: configs.c4_rownorm(be, o, x, g, b), reps=30))

    n5 = configs.C5_SHAPE[0] * configs.C5_SHAPE[1]
    line = (1, configs.C5_SHAPE[1])

    def make_c5(dtype):
        def make(k):
            x, idx = inputs("c5")
            if "i5" not in shared:
                shared["i5"] = be.array(idx, dtype=i32)
            return be.empty(line, dtype=dtype), be.array(roll(x, k))
        return make
    cases.append(Case("C5a argmax axis0 (32000,256) f32", configs.bytes_c5_reduce(), n5, make_c5(i32),
                      lambda o, x: configs.c5a_argmax(be, o, x)))
    cases.append(Case("C5b max axis0 (32000,256) f32", configs.bytes_c5_reduce(), n5, make_c5(f32),
                      lambda o, x: configs.c5b_max(be, o, x)))
    cases.append(Case("C5c cross-entropy axis0 (32000,256) f32, in-kernel one-hot", configs.bytes_c5c(), n5, make_c5(f32),
                      lambda o, x: configs.c5c_cross_entropy(be, o, x, be.onehot(shared["i5"], axis=0))))
    # floors of the latency-bound rows: what a launch, one trip to memory and back and (for the split
    # column reduction) the publish / ticket / fold hand-off cost when there is next to nothing to stream
    cases.append(Case("floor: elementwise kernel on 4 KB", 8192, 1024,
                      lambda k: (be.empty((1, 1024)), be.zeros((1, 1024))),
                      lambda o, x: o.__setitem__(slice(None), x * 2.0), cold=False))
    cases.append(Case("floor: split column max on 1 MB (8192,32)", 4 * 8192 * 32, 8192 * 32,
                      lambda k: (be.empty((1, 32)), be.zeros((8192, 32))),
                      lambda o, x: o.__setitem__(slice(None), be.max(x, axis=0)), cold=False))
    return cases


def case_plan(be, case, tensors):
    """the launch plan of a single-kernel case"""
    with be.capture() as grp:
        case.issue(*tensors)
    assert len(grp) == 1, "%s is not one kernel" % case.label
    _, plan = be.time_group(grp[0], reps=1)
    return plan


def gpu_leg(steps, warmup, detail=True, no_cold=False, hot_cold_only=False):
    from neon_amd import configs
    from neon_amd.backends import gen_backend
    from neon_amd.backends.backend import Block

    be = gen_backend("hip", rng_seed=0)
    be.bsz = 1
    rt = be.rt
    out = {"device": rt.props.name.decode(), "arch": rt.arch, "compute_units": be.cu_count}

    # ---- headline: fused Adam, full size, through the public API -----------------------
    grad_h, param_h = configs.inputs_c3()
    g, p = be.array(grad_h), be.array(param_h)
    m, v = be.zeros(configs.C3_SHAPE), be.zeros(configs.C3_SHAPE)
    del grad_h, param_h

    def adam_step(t):
        be.begin(Block.update, t)
        configs.c3_adam_step(be, p, g, m, v, t)
        be.end(Block.update, t)

    t = 0
    for _ in range(warmup):
        t += 1
        adam_step(t)
    be.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        t += 1
        adam_step(t)
    be.synchronize()
    wall = time.perf_counter() - t0
    step_bytes = configs.bytes_c3(fused=True)
    out["ms_per_step"] = wall * 1e3 / steps
    out["value_gbs"] = step_bytes * steps / wall / 1e9
    out["elements_per_s"] = configs.C3_SHAPE[0] * configs.C3_SHAPE[1] * steps / wall

    # the same kernel alone, HIP events around `steps` launches
    with be.capture() as groups:
        adam_step(t + 1)
    assert len(groups) == 1 and len(groups[0]) == 3, "Adam did not fuse into one kernel"
    ms, plan = be.time_group(groups[0], reps=max(steps, 5))
    out["roofline"] = {"bound": "hbm", "achieved": step_bytes / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS,
                       "unit": "GB/s", "frac": step_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                       "traffic": measured_traffic(plan.spec.name), "kernel": plan.spec.name, "kernel_ms": ms,
                       "kernel_us_rocprof": rocprof_us(plan.spec.name, "hot"), "algorithmic_bytes": step_bytes}
    if not detail:
        return out, be

    # ---- every configuration, kernel by kernel -------------------------------------------
    rows = []

    def api_ms(issue, reps):
        """wall-clock per call through the public API (host work included); three
        untimed calls first: a statement is recorded by its first call, gets its launch
        records with the second and is served by the C replayer from the third"""
        for _ in range(3):
            issue()
        be.synchronize()
        reps = max(reps, 200)
        t0 = time.perf_counter()
        for _ in range(reps):
            issue()
        be.synchronize()
        return (time.perf_counter() - t0) * 1e3 / reps

    def finish(row, nbytes, elements, mode="hot"):
        row["gbs"] = nbytes / (row["ms"] * 1e-3) / 1e9
        row["frac_of_hbm_peak"] = row["gbs"] / HBM_PEAK_GBS
        row["elements_per_s"] = elements / (row["ms"] * 1e-3) if elements else None
        # the same kernel's median duration in the committed rocprofv3 kernel trace (by kernel name)
        us = rocprof_us(row["kernel"], mode) if row.get("kernel") else None
        row["kernel_us_rocprof"] = us
        row["frac_rocprof"] = (nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS) if us else None
        row["traffic"] = measured_traffic(row["kernel"]) if row.get("kernel") else None
        rows.append(row)

    def measure(label, issue, nbytes, elements, reps=50):
        from neon_amd.backends.hip.planner import NeedsSplit
        from neon_amd.backends.hip.optree_ir import MixedAxes
        with be.capture() as grp:
            issue()
        row = {"config": label, "bytes": nbytes, "kernel": None}
        try:
            total, names, kernels = 0.0, [], []
            for trees in grp:
                ms_k, pl = be.time_group(trees, reps=reps)
                total += ms_k
                kernels.append(pl.spec.name)
                names.append("%s[%s]" % (pl.spec.family, ",".join(
                    "%s=%s" % kv for kv in sorted(pl.spec.params.items())
                    if kv[0] in ("V", "LX", "LY", "NCH", "NR"))))
            row.update({"kernels": len(grp), "ms": total, "timing": "HIP events around back-to-back launches",
                        "plan": " + ".join(names), "kernel": kernels[0] if len(kernels) == 1 else None})
        except (NeedsSplit, MixedAxes):
            before = be.plan_stats["launches"]
            issue()
            row["kernels"] = be.plan_stats["launches"] - before
            row["ms"] = api_ms(issue, reps)
            row["timing"] = "wall clock per API call (several kernels through temporaries)"
        row["api_ms"] = api_ms(issue, reps)
        finish(row, nbytes, elements)

    # the same trees with cold caches: each launch works on another set of tensors, enough sets
    # (>= 768 MB in total) that neither the L2s nor the 256 MB memory-side cache hold them
    def measure_cold(case):
        nsets = case.nsets()
        sets = [case.make(k) for k in range(nsets)]
        groups = []
        for tensors in sets:
            with be.capture() as grp:
                case.issue(*tensors)
            assert len(grp) == 1, "cold rows are single-kernel trees"
            groups.append(grp[0])
        be.time_group_sets(groups, reps=nsets)                    # touch every buffer once
        ms_k, pl = be.time_group_sets(groups, reps=max(2 * nsets, 60))
        finish({"config": case.label + " [cold]", "bytes": case.nbytes, "kernels": 1, "ms": ms_k, "api_ms": None,
                "timing": "HIP events around launches rotating over %d tensor sets of seeded random data" % nsets,
                "plan": pl.spec.family, "kernel": pl.spec.name}, case.nbytes, case.elements, mode="cold")
        del sets, groups

    for case in baseline_cases(be):
        if case.label.startswith("C3"):
            tensors = (p, g, m, v)          # the headline's tensors (400 MB) serve
        else:
            tensors = case.make(0)
        measure(case.label + ("" if case.nbytes > (256 << 20) or case.label.startswith("floor") else " [cache-hot]"),
                lambda: case.issue(*tensors), case.nbytes, case.elements, reps=case.reps)
        del tensors
        if case.cold and not no_cold:
            measure_cold(case)
    if hot_cold_only:
        out["per_config"] = rows
        return out, be

    rs = np.random.RandomState(11)
    n3 = configs.C3_SHAPE[0] * configs.C3_SHAPE[1]
    # the trees whose working set fits in cache, at >= 256 MB (what the same kernels do when bandwidth is the limit)
    big = (16384, 4096)   # 256 MiB per tensor
    xb, yb, ob = _fresh(be, big, rs=rs), _fresh(be, big, rs=rs), be.empty(big)
    nb = big[0] * big[1]
    measure("C1a scaled (16384,4096) f32", lambda: configs.c1a(be, ob, xb, yb), configs.bytes_c1a(big), nb, reps=10)
    measure("C1b scaled (16384,4096) f32", lambda: configs.c1b(be, ob), configs.bytes_c1b(big), nb, reps=10)
    del yb, xb
    wide = (1000, 65536)  # same depth, 512x the columns: 262 MB per tensor
    xw = _fresh(be, wide, rs=rs, scale=3.0)
    ow = ob.share(wide)
    measure("C2 softmax axis0 scaled (1000,65536) f32", lambda: configs.c2_softmax(be, ow, xw),
            configs.bytes_c2(wide), wide[0] * wide[1], reps=10)
    del xw, ow, ob
    # C3 as the API states it
    measure("C3 Adam as 3 assigns, 3 kernels (5000,5000) f32",
            lambda: configs.c3_adam_step(be, p, g, m, v, t + 2), configs.bytes_c3(fused=False), n3, reps=20)

    def adam_in_minibatch():
        # the optimizer's statements as written, inside the hint that the reference's
        # training loop puts round every minibatch (models/model.py:204-217)
        be.begin(Block.minibatch, 0)
        configs.c3_adam_step(be, p, g, m, v, t + 2)
        be.end(Block.minibatch, 0)
    measure("C3 Adam as 3 assigns inside a minibatch block (5000,5000) f32", adam_in_minibatch,
            configs.bytes_c3(fused=True), n3, reps=20)
    # C4 on bfloat16 storage; C5a and C5b in one launch
    from neon_amd.backends import bfloat16
    x4h, gh, bh = configs.inputs_c4()
    x4, o4 = be.array(x4h, dtype=np.float16), be.empty(configs.C4_SHAPE, dtype=np.float16)
    g4, b4 = be.array(gh), be.array(bh)
    del x4h
    x4b, o4b = be.empty(configs.C4_SHAPE, dtype=bfloat16), be.empty(configs.C4_SHAPE, dtype=bfloat16)
    x4b[:] = x4
    measure("C4 rownorm (256,100352) bf16", lambda: configs.c4_rownorm(be, o4b, x4b, g4, b4), configs.bytes_c4(),
            configs.C4_SHAPE[0] * configs.C4_SHAPE[1], reps=30)
    del x4b, o4b
    x5h, i5h = configs.inputs_c5()
    x5 = be.array(x5h)
    am = be.empty((1, configs.C5_SHAPE[1]), dtype=np.int32)
    mx = be.empty((1, configs.C5_SHAPE[1]))
    n5 = x5h.size
    del x5h

    def c5ab():
        with be.fused():
            configs.c5a_argmax(be, am, x5)
            configs.c5b_max(be, mx, x5)
    measure("C5a+b argmax and max in one launch (32000,256) f32", c5ab, configs.bytes_c5_reduce() + 4 * configs.C5_SHAPE[1], n5)
    # ---- the prebuilt hand-written kernels behind the direct C-ABI entry points ------------
    lib = rt.lib
    e0, e1 = rt.event(), rt.event()

    def measure_abi(label, part, call, nbytes, elements, reps=30):
        for _ in range(3):
            call()
        rt.synchronize()
        rt.event_record(e0)
        for _ in range(reps):
            rc = call()
        rt.event_record(e1)
        rt.event_sync(e1)
        assert rc == 0, lib.nh_last_error()
        ms_k = rt.event_elapsed_ms(e0, e1) / reps
        us = rocprof_us_part(part, "hot")
        rows.append({"config": label, "bytes": nbytes, "kernels": 1, "ms": ms_k, "api_ms": ms_k,
                     "timing": "HIP events around back-to-back C-ABI calls through ctypes: for a kernel of a few "
                               "microseconds this is the rate of the calls, not the kernel (see kernel_us_rocprof)",
                     "plan": "prebuilt (kernels.hip)",
                     "gbs": nbytes / (ms_k * 1e-3) / 1e9, "frac_of_hbm_peak": nbytes / (ms_k * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "elements_per_s": elements / (ms_k * 1e-3), "kernel_us_rocprof": us,
                     "frac_rocprof": (nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS) if us else None})

    measure_abi("C3 prebuilt nh_adam_step_f32 (5000,5000) f32", PREBUILT_PARTS["adam"],
                lambda: lib.nh_adam_step_f32(p.ptr, m.ptr, v.ptr, g.ptr, 1e-3, 0.9, 0.1, 0.999, 0.001, 1e-8, n3, None),
                configs.bytes_c3(fused=True), n3)
    measure_abi("C4 prebuilt nh_rownorm_f16 (256,100352) f16", PREBUILT_PARTS["rownorm"],
                lambda: lib.nh_rownorm_f16(o4.ptr, x4.ptr, g4.ptr, b4.ptr, 1e-5, configs.C4_SHAPE[0],
                                           configs.C4_SHAPE[1], configs.C4_SHAPE[1], None),
                configs.bytes_c4(), configs.C4_SHAPE[0] * configs.C4_SHAPE[1])
    ws = rt.malloc(lib.nh_colreduce_workspace_bytes(configs.C5_SHAPE[0], configs.C5_SHAPE[1]))
    measure_abi("C5a+b prebuilt nh_colmax_argmax_f32 (32000,256) f32", PREBUILT_PARTS["colmax"],
                lambda: lib.nh_colmax_argmax_f32(mx.ptr, am.ptr, x5.ptr, configs.C5_SHAPE[0], configs.C5_SHAPE[1],
                                                 configs.C5_SHAPE[1], ws, None),
                configs.bytes_c5_reduce() + 4 * configs.C5_SHAPE[1], n5)
    rt.synchronize()
    rt.free(ws)
    del x5, x4, o4
    next_rows(be, rows)
    out["per_config"] = rows
    return out, be


def next_rows(be, rows):
    """Callers either side of the op-tree path (batch norm, random numbers and
    rounding, indexing and layout, compensated accumulation, the GEMM
    hand-off), each on a shape of the benchmark configurations, timed like the
    rows above and priced by the bytes (or flops) the operation has to move."""
    rt = be.rt
    f32, f16, i32 = np.float32, np.float16, np.int32
    rs = np.random.RandomState(5)
    e0, e1 = rt.event(), rt.event()

    def add(label, ms_k, nbytes, plan, kernels=1, flops=None):
        row = {"config": label, "bytes": nbytes, "kernels": kernels, "ms": ms_k, "api_ms": None,
               "timing": "HIP events around back-to-back launches", "plan": plan,
               "gbs": nbytes / (ms_k * 1e-3) / 1e9, "frac_of_hbm_peak": nbytes / (ms_k * 1e-3) / 1e9 / HBM_PEAK_GBS,
               "elements_per_s": None}
        if flops:
            row["tflops"] = flops / (ms_k * 1e-3) / 1e12
        rows.append(row)

    def trees(label, issue, nbytes, reps=30):
        with be.capture() as grp:
            issue()
        total, names = 0.0, []
        for group in grp:
            ms_k, pl = be.time_group(group, reps=reps)
            total += ms_k
            names.append(pl.spec.family)
        add(label, total, nbytes, " + ".join(names), kernels=len(grp))

    def calls(label, call, nbytes, plan, reps=30, flops=None):
        for _ in range(3):
            call()
        rt.synchronize()
        rt.event_record(e0)
        for _ in range(reps):
            call()
        rt.event_record(e1)
        rt.event_sync(e1)
        add(label, rt.event_elapsed_ms(e0, e1) / reps, nbytes, plan, flops=flops)

    # batch norm over (256 feature maps, 100352 = N*H*W) fp16, as one fused kernel each way;
    # then the same bytes as 64 feature maps (an early convolution): four workgroups per row
    for K, N in ((256, 100352), (64, 401408)):
        x = _fresh(be, (K, N), dtype=f16, rs=rs, scale=2.0, shift=0.5)
        y = be.empty((K, N), dtype=f16)
        vec = lambda fill: _fresh(be, (K, 1), fill=fill)
        xsum, xvar, gmean, gvar, gamma, beta = vec(0.0), vec(0.0), vec(0.0), vec(1.0), vec(1.0), vec(0.0)
        trees("BN fprop fused (%d,%d) f16" % (K, N), lambda: be.compound_fprop_bn(
            x, xsum, xvar, gmean, gvar, gamma, beta, y, 1e-5, 0.9, True), 2 * K * N * 2)
        delta = _fresh(be, (K, N), dtype=f16, rs=rs, scale=0.1)
        dout = be.empty((K, N), dtype=f16)
        gg, gb = vec(0.0), vec(0.0)
        trees("BN bprop fused (%d,%d) f16" % (K, N), lambda: be.compound_bprop_bn(
            dout, gg, gb, delta, x, xsum, xvar, gamma, 1e-5), 3 * K * N * 2)
        del x, y, delta, dout

    # random numbers and rounding on the Adam shape
    shape = (5000, 5000)
    n = shape[0] * shape[1]
    a32, b32 = _fresh(be, shape, rs=rs), be.empty(shape)
    trees("dropout mask (5000,5000) f32", lambda: be.make_binary_mask(b32, 0.5), n * 4)
    trees("dropout applied x*mask/keep (5000,5000) f32",
          lambda: b32.__setitem__(slice(None), a32 * be.dropout(0.5) * 2.0), 2 * n * 4)
    r16 = be.empty(shape, dtype=f16)
    r16.rounding = 8
    trees("stochastic-rounding store f32 -> f16, 8 bits (5000,5000)",
          lambda: r16.__setitem__(slice(None), a32 * 1.0), n * 6)
    s16, c16, a16 = be.zeros(shape, dtype=f16), be.zeros(shape, dtype=f16), _fresh(be, shape, dtype=f16, rs=rs)
    calls("compensated_sum (5000,5000) f16", lambda: be.compensated_sum(s16, c16, a16), 5 * n * 2, "ew")
    del r16, s16, c16, a16

    # indexing and layout
    calls("hist log2 (5000,5000) f32", lambda: a32.hist("bench"), n * 4, "prebuilt (kernels.hip)")
    table = _fresh(be, (32000, 256), rs=rs)
    idx = be.array(rs.randint(0, 32000, size=(65536, 1)).astype(i32), dtype=i32)
    rows_out = be.empty((65536, 256))
    trees("gather 65536 rows of a (32000,256) f32 table", lambda: rows_out.__setitem__(slice(None), table[idx]),
          2 * 65536 * 256 * 4 + 65536 * 4)
    del table, rows_out, b32
    sq = (8192, 8192)
    t_in, t_out = _fresh(be, sq, rs=rs), be.empty(sq)
    calls("copy_transpose (8192,8192) f32", lambda: be.copy_transpose(t_in, t_out), 2 * sq[0] * sq[1] * 4,
          "prebuilt (kernels.hip)", reps=10)
    t3_in = t_in.reshape((64, 512, 2048))
    t3_out = t_out.reshape((2048, 64, 512))
    calls("copy_transpose (64,512,2048) f32 axes (2,0,1)", lambda: be.copy_transpose(t3_in, t3_out, axes=(2, 0, 1)),
          2 * sq[0] * sq[1] * 4, "prebuilt (kernels.hip)", reps=10)
    del t_in, t_out, t3_in, t3_out, a32
    h_in, h_out = _fresh(be, sq, dtype=f16, rs=rs), be.empty(sq, dtype=f16)
    calls("copy_transpose (8192,8192) f16", lambda: be.copy_transpose(h_in, h_out), 2 * sq[0] * sq[1] * 2,
          "prebuilt (kernels.hip)", reps=10)
    del h_in, h_out

    # the GEMM hand-off (library kernel; flops, not bytes, bound it)
    m = 4096
    for dt, label in ((f32, "f32"), (f16, "f16")):
        A, B, C = (_fresh(be, (m, m), dtype=dt, rs=rs, scale=0.1) for _ in range(3))
        calls("compound_dot (4096,4096)x(4096,4096) %s [library GEMM]" % label,
              lambda: be.compound_dot(A, B, C), 3 * m * m * np.dtype(dt).itemsize, "rocBLAS", reps=10,
              flops=2.0 * m * m * m)
        del A, B, C
    rt.synchronize()


def cpu_leg(max_seconds=25.0):
    """numpy oracle on the headline workload: full-size Adam steps, 1 core"""
    from neon_amd import configs
    from neon_amd.backends.backend import Backend
    from oracle import nervanacpu  # noqa: F401  (cpu_baseline leg only)
    cpu = Backend.allocate_backend("cpu", rng_seed=0)
    cpu.bsz = 1
    grad_h, param_h = configs.inputs_c3()
    g, p = cpu.array(grad_h), cpu.array(param_h)
    m, v = cpu.zeros(configs.C3_SHAPE), cpu.zeros(configs.C3_SHAPE)
    times = []
    t = 0
    t_begin = time.perf_counter()
    while True:
        t += 1
        t0 = time.perf_counter()
        configs.c3_adam_step(cpu, p, g, m, v, t)
        times.append(time.perf_counter() - t0)
        if len(times) >= 7 or (time.perf_counter() - t_begin) > max_seconds:
            break
    timed = times[1:] if len(times) > 2 else times      # first step pays page faults
    med = float(np.median(timed))
    try:
        with open("/proc/cpuinfo") as f:
            model = [l.split(":", 1)[1].strip() for l in f if l.startswith("model name")][0]
    except Exception:
        model = "unknown"
    del g, p, m, v, grad_h, param_h

    # the other configurations on the oracle, full size, median of 5 calls each (a few seconds in all)
    def median_s(issue, calls=5):
        issue()
        ts = []
        for _ in range(calls):
            t0 = time.perf_counter()
            issue()
            ts.append(time.perf_counter() - t0)
        return float(np.median(ts))

    per_config = []

    def row(label, issue, nbytes, elements):
        sec = median_s(issue)
        per_config.append({"config": label, "us": round(sec * 1e6, 1), "gbs": round(nbytes / sec / 1e9, 2),
                           "elements_per_s": elements / sec})

    x1, y1 = (cpu.array(a) for a in configs.inputs_c1())
    o1 = cpu.empty(configs.C1_SHAPE)
    n1 = configs.C1_SHAPE[0] * configs.C1_SHAPE[1]
    row("C1a", lambda: configs.c1a(cpu, o1, x1, y1), configs.bytes_c1a(), n1)
    row("C1b", lambda: configs.c1b(cpu, o1), configs.bytes_c1b(), n1)
    row("C1 fused", lambda: configs.c1_fused(cpu, o1, x1, y1), configs.bytes_c1a(), n1)
    x2, o2 = cpu.array(configs.inputs_c2()[0]), cpu.empty(configs.C2_SHAPE)
    row("C2", lambda: configs.c2_softmax(cpu, o2, x2), configs.bytes_c2(), configs.C2_SHAPE[0] * configs.C2_SHAPE[1])
    xh, gam, bet = configs.inputs_c4()
    # fp16 storage with fp32 arithmetic: the quantised values held as fp32, the result stored as fp16
    x4, g4, b4 = cpu.array(xh.astype(np.float32)), cpu.array(gam), cpu.array(bet)
    o4 = cpu.empty(configs.C4_SHAPE, dtype=np.float16)
    row("C4", lambda: configs.c4_rownorm(cpu, o4, x4, g4, b4), configs.bytes_c4(),
        configs.C4_SHAPE[0] * configs.C4_SHAPE[1])
    del x4, o4, xh
    x5h, idx = configs.inputs_c5()
    x5 = cpu.array(x5h)
    n5 = configs.C5_SHAPE[0] * configs.C5_SHAPE[1]
    am, mx, ce = (cpu.empty((1, configs.C5_SHAPE[1]), dtype=dt) for dt in (np.int32, np.float32, np.float32))
    row("C5a", lambda: configs.c5a_argmax(cpu, am, x5), configs.bytes_c5_reduce(), n5)
    row("C5b", lambda: configs.c5b_max(cpu, mx, x5), configs.bytes_c5_reduce(), n5)
    hot = cpu.empty(configs.C5_SHAPE)
    hot[:] = cpu.onehot(cpu.array(idx, dtype=np.int32), axis=0)      # the oracle takes the dense one-hot only
    row("C5c (dense one-hot)", lambda: configs.c5c_cross_entropy(cpu, ce, x5, hot), configs.bytes_c5c(), n5)
    return {"value": configs.bytes_c3(fused=True) / med / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "%d full-size Adam steps (5000x5000 fp32) on the numpy oracle, median step %.3f s; "
                      "numpy ufuncs are single-threaded" % (len(timed), med),
            "elements_per_s": configs.C3_SHAPE[0] * configs.C3_SHAPE[1] / med,
            "host_cpu": model, "host_cpu_count": os.cpu_count(), "per_config": per_config}


def counter_pass():
    """A short, untimed run for hardware-counter collection
    (``rocprofv3 --pmc FETCH_SIZE -- python3 bench.py --counter-pass``, then the
    same with WRITE_SIZE, or with SQ_* counters): three launches each of a
    plain copy kernel of known size (the calibration: 100 MB read, 100 MB
    written) and of the kernel behind every benchmark configuration and the
    batch-norm pair.  Prints which kernel belongs to which configuration and
    its algorithmic bytes (the table ``neon_amd.profile_summary`` joins with
    the counter files)."""
    from neon_amd import configs
    from neon_amd.backends import gen_backend
    be = gen_backend("hip", rng_seed=0)
    be.bsz = 1
    rs = np.random.RandomState(3)
    f16 = np.float16
    table = []

    def run(label, nbytes, issue, reps=3):
        with be.capture() as grp:
            issue()
        assert len(grp) == 1, label
        _, plan = be.time_group(grp[0], reps=1)
        for _ in range(reps):
            issue()
            be.synchronize()
        table.append({"label": label, "kernel": plan.spec.name, "family": plan.spec.family,
                      "algorithmic_bytes": nbytes, "warmup": 0, "launches": reps + 1})

    src = _fresh(be, configs.C3_SHAPE, rs=rs, scale=1e-2)
    dst = be.empty(configs.C3_SHAPE)
    run("copy (calibration)", 200000000, lambda: dst.__setitem__(slice(None), src * 1.0))
    del src, dst
    for case in baseline_cases(be):
        if case.label.startswith("floor"):
            continue
        tensors = case.make(0)
        run(case.label, case.nbytes, lambda: case.issue(*tensors))
        del tensors
    K, N = configs.C4_SHAPE
    x4 = _fresh(be, configs.C4_SHAPE, dtype=f16, rs=rs, scale=2.0, shift=0.5)
    o4 = be.empty(configs.C4_SHAPE, dtype=f16)
    vec = lambda fill: _fresh(be, (K, 1), fill=fill)
    xsum, xvar, gmean, gvar, gamma, beta = vec(0.0), vec(0.0), vec(0.0), vec(1.0), vec(1.0), vec(0.0)
    run("BN fprop (256,100352) f16", 2 * K * N * 2,
        lambda: be.compound_fprop_bn(x4, xsum, xvar, gmean, gvar, gamma, beta, o4, 1e-5, 0.9, True))
    delta = _fresh(be, (K, N), dtype=f16, rs=rs, scale=0.1)
    gg, gb = vec(0.0), vec(0.0)
    run("BN bprop (256,100352) f16", 3 * K * N * 2,
        lambda: be.compound_bprop_bn(o4, gg, gb, delta, x4, xsum, xvar, gamma, 1e-5))
    del x4, o4, delta

    # the two prebuilt kernels that go through LDS (their names are the compiler's: matched by a part)
    def run_prebuilt(label, part, nbytes, call, reps=3):
        for _ in range(reps + 1):
            call()
            be.synchronize()
        table.append({"label": label, "kernel": None, "kernel_contains": part, "family": "prebuilt",
                      "algorithmic_bytes": nbytes, "warmup": 0, "launches": reps + 1})
    a32 = _fresh(be, configs.C3_SHAPE, rs=rs)
    run_prebuilt("hist log2 (5000,5000) f32", "hist_", a32.size * 4, lambda: a32.hist("bench"))
    sq = (8192, 8192)
    t_in, t_out = _fresh(be, sq, rs=rs), be.empty(sq)
    run_prebuilt("copy_transpose (8192,8192) f32", "transpose_tile", 2 * sq[0] * sq[1] * 4,
                 lambda: be.copy_transpose(t_in, t_out))
    print(json.dumps({"pass": "counters", "rows": table}))


TRACE_WARMUP, TRACE_LAUNCHES = 12, 60
# a part of the compiler's name for each prebuilt kernel behind a direct C-ABI entry point
PREBUILT_PARTS = {"adam": "AdamF", "rownorm": "rownorm_f16_kernel", "colmax": "colmax_kernel"}


def trace_pass(mode):
    """The program behind the kernel-duration summaries
    (``rocprofv3 --kernel-trace -- python3 bench.py --trace-pass hot``, then
    ``cold``): for every benchmark configuration TRACE_WARMUP warm-up launches
    and TRACE_LAUNCHES measured ones of its kernel, through the public API --
    ``hot`` on one set of tensors, ``cold`` rotating over enough sets (>= 768 MB
    of seeded random data) that no launch finds its operands in a cache, every
    set touched during the warm-up.  Prints the table that
    ``neon_amd.profile_summary durations`` joins with the trace."""
    from neon_amd.backends import gen_backend
    be = gen_backend("hip", rng_seed=0)
    be.bsz = 1
    table = []
    for case in baseline_cases(be):
        if mode == "cold" and not case.cold:
            continue
        nsets = case.nsets() if mode == "cold" else 1
        sets = [case.make(k) for k in range(nsets)]
        plan = case_plan(be, case, sets[0])
        warm = max(TRACE_WARMUP, nsets)
        for i in range(warm + TRACE_LAUNCHES):
            case.issue(*sets[i % nsets])
        be.synchronize()
        table.append({"label": case.label + (" [cold, %d sets]" % nsets if mode == "cold" else ""),
                      "kernel": plan.spec.name, "family": plan.spec.family, "algorithmic_bytes": case.nbytes,
                      "warmup": warm + 1, "launches": TRACE_LAUNCHES})        # (+1: the launch that made the plan)
        del sets
    if mode == "hot":
        _trace_support_rows(be, table)
    what = ("every launch on the same tensors (cache-hot where the working set fits a cache)" if mode == "hot" else
            "launches rotating over >= 768 MB of distinct tensor sets (cold caches)")
    note = ("Back-to-back launches through the public API, no synchronisation in between." if mode == "hot" else
            "Sets hold the configuration's seeded inputs rolled by 13 rows per set: random data in every launch.")
    print(json.dumps({"pass": mode, "what": what, "note": note, "rows": table}))


def _trace_support_rows(be, table):
    """hot-pass rows beyond the benchmark configurations: the batch-norm pair on both of its
    shapes (one workgroup per row, and several cooperating workgroups per row), softmax down
    cooperating column strips, the two prebuilt kernels that stage data in LDS, and the
    hand-written kernels behind the direct C-ABI entry points of C3, C4 and C5"""
    from neon_amd import configs
    rs = np.random.RandomState(3)
    f16 = np.float16

    def generated(label, nbytes, issue):
        with be.capture() as grp:
            issue()
        assert len(grp) == 1, label
        _, plan = be.time_group(grp[0], reps=1)
        for _ in range(TRACE_WARMUP + TRACE_LAUNCHES):
            issue()
        be.synchronize()
        table.append({"label": label, "kernel": plan.spec.name, "family": plan.spec.family, "algorithmic_bytes": nbytes,
                      "warmup": TRACE_WARMUP + 1, "launches": TRACE_LAUNCHES})   # (+1: the launch that made the plan)

    def prebuilt(label, part, nbytes, call):
        for _ in range(TRACE_WARMUP + TRACE_LAUNCHES):
            call()
        be.synchronize()
        table.append({"label": label, "kernel": None, "kernel_contains": part, "family": "prebuilt",
                      "algorithmic_bytes": nbytes, "warmup": TRACE_WARMUP, "launches": TRACE_LAUNCHES})

    for K, N in (configs.C4_SHAPE, (64, 401408)):
        x = _fresh(be, (K, N), dtype=f16, rs=rs, scale=2.0, shift=0.5)
        y = be.empty((K, N), dtype=f16)
        vec = lambda fill: _fresh(be, (K, 1), fill=fill)
        xsum, xvar, gmean, gvar, gamma, beta = vec(0.0), vec(0.0), vec(0.0), vec(1.0), vec(1.0), vec(0.0)
        generated("BN fprop (%d,%d) f16" % (K, N), 2 * K * N * 2,
                  lambda: be.compound_fprop_bn(x, xsum, xvar, gmean, gvar, gamma, beta, y, 1e-5, 0.9, True))
        delta = _fresh(be, (K, N), dtype=f16, rs=rs, scale=0.1)
        dout, gg, gb = be.empty((K, N), dtype=f16), vec(0.0), vec(0.0)
        generated("BN bprop (%d,%d) f16" % (K, N), 3 * K * N * 2,
                  lambda: be.compound_bprop_bn(dout, gg, gb, delta, x, xsum, xvar, gamma, 1e-5))
        del x, y, delta, dout
    xs = _fresh(be, configs.C5_SHAPE, rs=rs)
    ys = be.empty(configs.C5_SHAPE)
    generated("softmax axis0 (32000,256) f32", 2 * xs.size * 4, lambda: configs.c2_softmax(be, ys, xs))
    del xs, ys
    a32 = _fresh(be, configs.C3_SHAPE, rs=rs)
    prebuilt("hist log2 (5000,5000) f32", "hist_", a32.size * 4, lambda: a32.hist("bench"))
    del a32
    sq = (8192, 8192)
    t_in, t_out = _fresh(be, sq, rs=rs), be.empty(sq)
    prebuilt("copy_transpose (8192,8192) f32", "transpose_tile", 2 * sq[0] * sq[1] * 4,
             lambda: be.copy_transpose(t_in, t_out))
    del t_in, t_out
    # the hand-written kernels behind the direct C-ABI entry points of three configurations
    lib = be.rt.lib
    n3 = configs.C3_SHAPE[0] * configs.C3_SHAPE[1]
    p, m, v, g = (_fresh(be, configs.C3_SHAPE, rs=rs, scale=1e-2) for _ in range(4))
    prebuilt("C3 prebuilt nh_adam_step_f32 (5000,5000) f32", PREBUILT_PARTS["adam"], configs.bytes_c3(fused=True),
             lambda: lib.nh_adam_step_f32(p.ptr, m.ptr, v.ptr, g.ptr, 1e-3, 0.9, 0.1, 0.999, 0.001, 1e-8, n3, None))
    del p, m, v, g
    K, N = configs.C4_SHAPE
    x4 = _fresh(be, (K, N), dtype=f16, rs=rs, scale=2.0, shift=0.5)
    o4, g4, b4 = be.empty((K, N), dtype=f16), _fresh(be, (K, 1), fill=1.0), _fresh(be, (K, 1), fill=0.0)
    prebuilt("C4 prebuilt nh_rownorm_f16 (256,100352) f16", PREBUILT_PARTS["rownorm"], configs.bytes_c4(),
             lambda: lib.nh_rownorm_f16(o4.ptr, x4.ptr, g4.ptr, b4.ptr, 1e-5, K, N, N, None))
    del x4, o4
    R5, C5 = configs.C5_SHAPE
    x5, mx, am = _fresh(be, (R5, C5), rs=rs), be.empty((1, C5)), be.empty((1, C5), dtype=np.int32)
    ws = be.rt.malloc(lib.nh_colreduce_workspace_bytes(R5, C5))
    prebuilt("C5a+b prebuilt nh_colmax_argmax_f32 (32000,256) f32", PREBUILT_PARTS["colmax"],
             configs.bytes_c5_reduce() + 4 * C5,
             lambda: lib.nh_colmax_argmax_f32(mx.ptr, am.ptr, x5.ptr, R5, C5, C5, ws, None))
    be.rt.free(ws)


def shape_sweep(dtype_name):
    """Seven common trees over a grid of shapes between 8 MB and 1 GB: wall
    clock per call through the public API, and the fraction of the HBM peak
    the algorithmic bytes come to.  A map of where the kernel families stand
    away from the five benchmark shapes (``python bench.py --sweep float32``)."""
    from neon_amd.backends import gen_backend
    be = gen_backend("hip", rng_seed=0)
    dt = np.dtype(dtype_name)
    isz = dt.itemsize

    def per_call_us(issue, reps):
        for _ in range(3):
            issue()
        be.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            issue()
        be.synchronize()
        return (time.perf_counter() - t0) * 1e6 / reps

    names = ("x*2+1", "x+col", "sum ax0", "sum ax1", "argmax ax0", "softmax ax0", "softmax ax1")
    print("%s storage; cells: microseconds per call / fraction of %.0f GB/s" % (dt.name, HBM_PEAK_GBS))
    print("%-18s %s" % ("shape", " ".join("%12s" % n for n in names)))
    dims = (64, 1000, 4096, 30000, 131072, 1048576)
    for R in dims:
        for C in dims:
            n = R * C
            if n * isz < (8 << 20) or n * isz > (1 << 30):
                continue
            x, o = be.empty((R, C), dtype=dt), be.empty((R, C), dtype=dt)
            x[:] = be.rand()
            col, row, irow = be.zeros((R, 1)), be.zeros((1, C)), be.zeros((1, C), dtype=np.int32)
            reps = max(3, min(50, int(2e9 / (n * isz))))
            trees = (
                (lambda: o.__setitem__(slice(None), x * 2.0 + 1.0), 2),
                (lambda: o.__setitem__(slice(None), x + col), 2),
                (lambda: row.__setitem__(slice(None), be.sum(x, axis=0)), 1),
                (lambda: col.__setitem__(slice(None), be.sum(x, axis=1)), 1),
                (lambda: irow.__setitem__(slice(None), be.argmax(x, axis=0)), 1),
                (lambda: o.__setitem__(slice(None), be.exp(x - be.max(x, axis=0)) /
                                       be.sum(be.exp(x - be.max(x, axis=0)), axis=0)), 2),
                (lambda: o.__setitem__(slice(None), be.exp(x - be.max(x, axis=1)) /
                                       be.sum(be.exp(x - be.max(x, axis=1)), axis=1)), 2))
            cells = []
            for issue, passes in trees:
                us = per_call_us(issue, reps)
                cells.append("%6.0f/%.2f" % (us, passes * n * isz / us / 1e3 / HBM_PEAK_GBS))
            print("%-18s %s" % ((R, C), " ".join("%12s" % c for c in cells)), flush=True)
            del x, o


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-oracle leg")
    ap.add_argument("--no-detail", action="store_true", help="headline only, no per-config table")
    ap.add_argument("--counter-pass", action="store_true",
                    help="short untimed run for rocprofv3 --pmc (see counter_pass)")
    ap.add_argument("--trace-pass", choices=("hot", "cold"), default=None,
                    help="the launches a rocprofv3 --kernel-trace run summarises (see trace_pass)")
    ap.add_argument("--no-cold", action="store_true", help="skip the cold-cache rows")
    ap.add_argument("--configs-only", action="store_true",
                    help="headline + the benchmark configurations (hot and cold), none of the widened rows")
    ap.add_argument("--sweep", metavar="DTYPE", default=None,
                    help="common trees over a grid of shapes (float32 / float16), see shape_sweep")
    args = ap.parse_args()
    if args.sweep:
        import __graft_entry__
        __graft_entry__.ensure_built()
        shape_sweep(args.sweep)
        return
    if args.counter_pass or args.trace_pass:
        import __graft_entry__
        __graft_entry__.ensure_built()
        if args.counter_pass:
            counter_pass()
        else:
            trace_pass(args.trace_pass)
        return
    if args.gpus != 1:
        print("bench.py measures one MI355X; --gpus %d is not supported (the op-tree path has no "
              "cross-device stage: every figure here is one GPU's)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import __graft_entry__
    __graft_entry__.ensure_built()
    gpu, be = gpu_leg(args.steps, args.warmup, detail=not args.no_detail, no_cold=args.no_cold,
                      hot_cold_only=args.configs_only)
    cpu = None if args.no_cpu else cpu_leg()
    line = {
        "metric": "fused op-tree HBM GB/s (% of MI355X peak) + elements/s vs CPU backend",
        "value": gpu["value_gbs"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": gpu["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "C3: fused Adam update op-tree, 25,000,000 fp32 params (5000x5000), "
                               "4 tensors read + 3 written per step, lr=1e-3 b1=0.9 b2=0.999 eps=1e-8",
                   "algorithmic_bytes_per_step": 700000000, "parallelism": "single GPU"},
        "frac_of_hbm_peak": gpu["value_gbs"] / HBM_PEAK_GBS,
        "elements_per_s": gpu["elements_per_s"],
        "roofline": gpu["roofline"],
        "cpu_baseline": cpu,
        "device": gpu["device"], "arch": gpu["arch"],
    }
    if cpu:
        line["gpu_over_cpu"] = gpu["value_gbs"] / cpu["value"]
    per_config = gpu.get("per_config")
    if per_config:
        def short(r):
            d = {"config": r["config"], "us": round(r["ms"] * 1e3, 3),
                 "api_us": round(r["api_ms"] * 1e3, 3) if r.get("api_ms") else None,
                 "bytes": r["bytes"], "gbs": round(r["gbs"], 1), "frac": round(r["frac_of_hbm_peak"], 4),
                 "kernels": r["kernels"], "plan": r["plan"].split("[")[0] if "+" not in r["plan"] else r["plan"]}
            if r.get("kernel"):
                d["kernel"] = r["kernel"]
                d["kernel_us_rocprof"] = r.get("kernel_us_rocprof")
                d["frac_rocprof"] = round(r["frac_rocprof"], 4) if r.get("frac_rocprof") else None
                d["traffic"] = r.get("traffic")
            elif r.get("kernel_us_rocprof"):           # a prebuilt kernel, found by a part of its name
                d["kernel_us_rocprof"] = r["kernel_us_rocprof"]
                d["frac_rocprof"] = round(r["frac_rocprof"], 4)
            return d
        line["per_config"] = [short(r) for r in per_config]
    print(json.dumps(line))
    sys.stdout.flush()
    if per_config:
        # The readable table goes to stderr AFTER the JSON line, the benchmark configurations last, so that
        # a reader who keeps only the end of the output still has them.  `events us` = HIP events around
        # back-to-back launches (includes the dispatch gap between launches); `rocprof us` = median kernel
        # duration of the same kernel (by name) in the committed rocprofv3 kernel trace, `-` when the
        # committed summary was made from another version of the kernel.
        fmt = "%-68s %9s %8s %10s %8s %8s  %s"
        named = lambda r: r["config"][:2] in ("C1", "C2", "C3", "C4", "C5") and "scaled" not in r["config"] \
            and "prebuilt" not in r["config"] and "bf16" not in r["config"] and "assigns" not in r["config"] \
            and "C5a+b" not in r["config"]
        for title, sel in (("operations around the path, scaled instances, prebuilt entry points", lambda r: not named(r)),
                           ("benchmark configurations (fractions of 8 TB/s on algorithmic bytes)", named)):
            print("\n" + title, file=sys.stderr)
            print(fmt % ("config", "events us", "of peak", "rocprof us", "of peak", "API us", "plan"), file=sys.stderr)
            for r in per_config:
                if not sel(r):
                    continue
                ru, rf = r.get("kernel_us_rocprof"), r.get("frac_rocprof")
                print(fmt % (r["config"][:68], "%.2f" % (r["ms"] * 1e3), "%.3f" % r["frac_of_hbm_peak"],
                             ("%.2f" % ru) if ru else "-", ("%.3f" % rf) if rf else "-",
                             ("%.2f" % (r["api_ms"] * 1e3)) if r.get("api_ms") else "-", r["plan"][:40]), file=sys.stderr)
        sys.stderr.flush()


if __name__ == "__main__":
    main()
