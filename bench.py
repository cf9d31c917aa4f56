#!/usr/bin/env python3
"""Benchmark of the layer-wise DP hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2|cfg3|cfg0|cfg1|cfg4|galvatron_like]

One "step" is one complete solve of the workload on the device: every layer's relaxation kernel
over every instance of the batch, plus the on-device backtrack, with the inputs already resident
in HBM (``gdp_plan_create`` has run).  Prints ONE JSON line.

* ``value``        min-plus relaxations per second, sum over instances of L*V*S*S divided by the
                   wall time of the timed steps (host clock around K steps, device synchronised on
                   both sides).  The timed solves carry out EVERY one of the L*V*S*S relaxations
                   (GDP_COMPUTE_ALL); ``with_row_skipping`` reports the library's default, which
                   skips rows it can prove irrelevant and returns identical results.
* ``roofline``     for the relaxation kernel (the only kernel that matters): the fp64 vector
                   operations the kernel needs AND ISSUES for the relaxations it carries out -- one
                   addition and one minimum per relaxation plus one addition per cell, 2 + 1/S (intra
                   is added after the minimum, which is exact because rounding is monotone); four per
                   relaxation where the argmin table is stored (two additions, compare, minimum; the
                   select beside them is a 32-bit operation) -- divided by the average launch duration measured with HIP events on the
                   stream the kernel runs on; peak = 39.3 T operations/s = MI355X's published
                   78.6 TFLOP/s fp64 vector rate, which counts an FMA as two operations (additions and
                   minima cannot fuse) at the published 2.4 GHz.  ``frac`` is therefore a fraction of
                   the instruction-issue roof and cannot exceed 1.  ``frac_reference_ops`` counts the 3
                   operations per relaxation of the reference's loop body (two additions and one
                   comparison, csrc/dp_core.cpp:65-73) over the same time: it can exceed 1, because the
                   kernel does not execute that work.  ``clock_ghz_under_load`` is the shader clock the
                   cycle counters in profiles/ give for this kernel under this workload (GRBM_GUI_ACTIVE
                   over the dispatch duration; null where not profiled): the peak assumes 2.4 GHz.
                   ``traffic`` is the measured HBM-side byte count per launch from profiles/, given
                   only while the kernel sources still hash to what was profiled.
* ``vs_baseline``  null: the reference publishes no number for this path.  ``vs_cpu_baseline_same_run`` is
                   ``value`` over ``cpu_baseline.value``: the reference's own code on ONE core of this host, timed
                   in this run -- a measured companion figure, not a published baseline.
* ``also.sweep_llama_like``  a whole search as the engine runs it (``SearchEngine.parallelism_optimization``,
                   the counterpart of search_engine.py:339-537, on a synthetic llama-like profile): all DP
                   instances of all tasks in one device batch.  Wall time of the call, the device's share (HIP
                   events around the kernels of every part of the batch, summed), the host's share (cost models,
                   input assembly, layout, copies: the rest), the relaxations of the mixed-shape batch and their
                   rate against the roofs, and whether the results equal the ones recorded from the reference's
                   engine (tests/golden/sweep_golden.json).
* ``also``         the other workloads, shorter legs, each with its own fractions and a ``bit_exact``
                   flag: results compared, outside the timed region, with the committed vectors
                   written from the reference's compiled dp_core (tests/golden/dp_core_golden.json).
                   ``roofline_hbm`` is the same launch against 8 TB/s with the algorithmic bytes
                   V*S*(8 read + 8 write) per layer and instance (the relaxation stores costs only;
                   the backtrack recomputes the argmin of the L cells on its path.  ``with_mark_table``
                   reports the mode that stores the reference's argmin table instead: 17 bytes and
                   five instead of two vector instructions per relaxation).
* ``config.plugin_call_ms``  one call of the drop-in ``galvatron_dp_core.dynamic_programming_core`` with the
                   reference's eleven arguments (single instances; median of a few calls).
* ``config.search_wall_ms_from_host_arrays``  the same solve through gdp_solve_batch from host arrays
                   (validation, layout, upload, all kernels, download; median of a few calls), beside
                   ``search_wall_ms_device`` (first kernel to last kernel of one solve, HIP events).
* ``cpu_baseline`` the reference's own dp_core (compiled into oracle/_ref by oracle/build.py) or,
                   where that file is absent, the C restatement in oracle/, timed on this host on a
                   bounded sample of the same workload (its first layers), one thread -- as the reference
                   runs.  ``also.cfg3.cpu_baseline_all_cores``: the 256 instances are independent, so
                   the C restatement is also timed with one thread per host core.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "hetu-galvatron_amd"))

PEAK_FP64_VALU_TFLOPS = 39.3   # 78.6 TFLOP/s published (FMA = 2 ops) / 2
PEAK_HBM_GBS = 8000.0
# Bytes per launch of the relaxation kernel between the L2s and the fabric (HBM and the memory-side
# cache in front of it), measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE and scaled by a copy
# kernel of known size; see profiles/.  Each figure belongs to the kernel sources it was measured on
# (first 16 hex digits of the SHA-256 of gdp_kernels.hip + gdp_kernels.h) and to one register tile; the
# bench line carries it only while both still match, null otherwise.
MEASURED_TRAFFIC = {
    # workload (+ mode): (bytes per launch, kernel sources hash, register tile "TSxR", profile)
    "cfg2": (12.131e9, "5abdfea757d76060", "16x1", "profiles/gdp_relax_fused_kernel_cfg2.txt"),                 # algorithmic 10.737e9
    "cfg2+row_skipping": (7.657e9, "5abdfea757d76060", "16x1", "profiles/gdp_relax_fused_kernel_cfg2_row_skipping.txt"),
    "cfg2+mark_table": (12.210e9, "5abdfea757d76060", "8x2", "profiles/gdp_relax_fused_kernel_cfg2_mark_table.txt"),  # algorithmic 11.409e9
    "cfg3": (45.78e9, "5abdfea757d76060", "15x3", "profiles/gdp_relax_fused_kernel_cfg3.txt"),   # algorithmic 44.3e9; average of the 4 launches of a solve
    "cfg4": (17.615e9, "5abdfea757d76060", "15x3", "profiles/gdp_relax_fused_kernel_cfg4.txt"),                 # algorithmic 17.716e9
}
KERNEL_SOURCES = ("hetu-galvatron_amd/csrc/gdp_kernels.hip", "hetu-galvatron_amd/csrc/gdp_kernels.h")
GOLDEN = os.path.join(ROOT, "tests", "golden", "dp_core_golden.json")


def _kernel_sources_hash() -> str:
    import hashlib
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def _traffic(key: str, tile: str):
    rec = MEASURED_TRAFFIC.get(key)
    if rec is None:
        return None, "not measured for this workload"
    nbytes, src_hash, rec_tile, profile = rec
    if src_hash != _kernel_sources_hash() or rec_tile != tile:
        return None, f"{profile} was measured on other kernel sources or another register tile"
    return nbytes, profile


# Shader clock under the relaxation kernel's load, from the cycle counters in profiles/ (GRBM_GUI_ACTIVE
# over the dispatch duration): the published peak assumes 2.4 GHz.
PROFILED_CLOCK_GHZ = {"cfg2": 2.14, "cfg3": 2.24, "cfg4": 2.29}


def _bit_exact(workload: str, probs) -> bool | None:
    """Results of the solved problems against the committed vectors written from the reference's
    compiled dp_core; None when the file or the case is absent."""
    if not os.path.exists(GOLDEN):
        return None
    with open(GOLDEN) as fh:
        golden = json.load(fh)
    names = [f"cfg3_{n:03d}" for n in range(len(probs))] if workload == "cfg3" else [workload]
    import numpy as np
    for name, prob in zip(names, probs):
        rec = golden.get(name)
        if rec is None:
            return None
        total = np.array([float.fromhex(h) for h in rec["total_hex"]])
        if total.tobytes() != prob.total.tobytes() or list(prob.remaining) != list(rec["remaining"]):
            return False
        for k, want in enumerate(rec["res"]):
            if prob.remaining[k] != -1 and [int(x) for x in prob.res[k]] != list(want):
                return False
    return True


def _problems(workload: str, compute_all: bool = True, keep_marks: bool = False):
    from galvatron_dp import _lib, workloads as W
    if workload == "cfg3":
        insts = W.config3()
    elif workload == "galvatron_like":
        insts = [W.galvatron_like()]      # the shape of one DPAlg.fit call of a real search (L=28, S=40, V=29493)
    else:
        insts = [W.CONFIGS[int(workload[3:])]()]
    probs = []
    for inst in insts:
        keys = sorted(inst.other_mem)
        probs.append(_lib.Problem(inst.mem, inst.intra, inst.inter_tables, inst.V,
                                  [inst.other_mem[k] for k in keys], [inst.other_time[k] for k in keys],
                                  inter_index=inst.inter_index, compute_all=compute_all,
                                  keep_marks=keep_marks))
    return insts, probs


def _host_description():
    """CPU model and number of logical processors of this host (for the CPU baseline figures)."""
    model = None
    try:
        with open("/proc/cpuinfo") as fh:
            for ln in fh:
                if ln.lower().startswith("model name"):
                    model = ln.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"cpu_model": model, "nproc": os.cpu_count()}


def _sweep_leg(name: str = "llama_like", repeats: int = 3):
    """One whole search through ``galvatron_dp.search.SearchEngine`` (scenario ``name`` of tests/sweep_cases.py: a
    synthetic profile, the argument records handed in); median of ``repeats`` runs after one untimed run."""
    import tempfile

    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import sweep_cases as S
    from galvatron_dp import _lib, cost_models
    from galvatron_dp.search import SearchEngine
    runs = []
    summary = None
    for rep in range(repeats + 1):
        with tempfile.TemporaryDirectory() as wd:
            eng = S.build(SearchEngine, cost_models, name, wd)
            eng.keep_device_cache = True                  # as inside a search service: allocations are reused
            _lib.batch_stats_begin()
            t0 = time.perf_counter()
            thr = eng.parallelism_optimization()
            wall = (time.perf_counter() - t0) * 1e3
            st = _lib.batch_stats_end()
            if rep == 0:
                summary = S.summarize(eng, thr, wd)
                continue
            runs.append((wall, st, eng.solved_instances))
    _lib.cache_trim()
    runs.sort(key=lambda r: r[0])
    wall, st, n_inst = runs[len(runs) // 2]
    bit_exact = None
    gpath = os.path.join(ROOT, "tests", "golden", "sweep_golden.json")
    if os.path.exists(gpath):
        with open(gpath) as fh:
            ref = json.load(fh)["sweeps"].get(name)
        if ref is not None:
            bit_exact = (summary["throughput"] == ref["throughput"] and summary["files"] == ref["files"] and
                         summary["table"] == ref["table"])
    dev_s = st.device_ms * 1e-3
    return {"scenario": name, "dp_instances": int(n_inst), "tasks_results": len(summary["table"]),
            "search_wall_ms": wall, "device_busy_ms": st.device_ms, "host_ms": wall - st.device_ms,
            "relaxations": st.relaxations, "relaxations_executed_fraction": st.executed / max(st.relaxations, 1.0),
            "value_wall": st.relaxations / (wall * 1e-3), "value_device": st.relaxations / max(dev_s, 1e-12),
            "roofline_frac_valu_fp64_device": 2.0 * st.executed / max(dev_s, 1e-12) / 1e12 / PEAK_FP64_VALU_TFLOPS,
            "batch_parts": int(st.parts), "parts_by_launch_scheme": {"flow": int(st.flow_parts), "fused": int(st.fused_parts),
                                                                      "per_layer": int(st.per_layer_parts)},
            "bit_exact": bit_exact}


def _cpu_baseline(workload: str, budget_s: float = 15.0):
    """Reference dp_core (or the C port) on the first layers of the workload's first instance."""
    import numpy as np
    from galvatron_dp import workloads as W
    from oracle import dp_oracle as O
    inst = (W.config3(n_limit=1)[0] if workload == "cfg3" else W.galvatron_like() if workload == "galvatron_like"
            else W.CONFIGS[int(workload[3:])]())
    use_ref = O.ref_available()
    fn = O.ref_solve if use_ref else O.solve
    per_layer = inst.V * inst.S * inst.S
    # one layer first to learn this host's rate, then as many layers as fit the time budget
    t0 = time.perf_counter()
    fn(inst.mem[:1], inst.intra[:1], np.ascontiguousarray(inst.inter[:1]), inst.V, inst.other_mem, inst.other_time)
    rate = per_layer / (time.perf_counter() - t0)
    n_layers = int(max(1, min(inst.L, budget_s * rate // per_layer)))
    mem, intra, inter = inst.mem[:n_layers], inst.intra[:n_layers], np.ascontiguousarray(inst.inter[:n_layers])
    t0 = time.perf_counter()
    fn(mem, intra, inter, inst.V, inst.other_mem, inst.other_time)
    dt = time.perf_counter() - t0
    relax = n_layers * per_layer
    return {"value": relax / dt, "unit": "relaxations/s", "cores": 1, **_host_description(),
            "kind": "reference" if use_ref else "port",
            "sample": f"first {n_layers} of {inst.L} layers of {inst.name} (V={inst.V}, S={inst.S}), "
                      f"{relax:.3g} relaxations in {dt:.2f} s, single thread, includes the host argmin-table "
                      f"allocation the reference caller does"}


def _cpu_baseline_all_cores(budget_s: float = 8.0):
    """cfg3's instances are independent: the C restatement of the reference (its ctypes call releases
    the interpreter lock) on one thread per host core, each solving the first layers of instances of
    the batch, for about ``budget_s`` seconds."""
    from concurrent.futures import ThreadPoolExecutor

    import numpy as np
    from galvatron_dp import workloads as W
    from oracle import dp_oracle as O
    cores = int(os.environ.get("OMP_NUM_THREADS") or 0) or min(16, os.cpu_count() or 1)
    insts = W.config3(n_limit=cores)
    n_layers = 2

    def one(inst):
        k = min(n_layers, inst.L)
        O.solve(inst.mem[:k], inst.intra[:k], np.ascontiguousarray(inst.inter[:k]), inst.V, inst.other_mem, inst.other_time)
        return float(k) * inst.V * inst.S * inst.S

    with ThreadPoolExecutor(cores) as pool:
        list(pool.map(one, insts[:cores]))                  # page in, learn the rate
        t0 = time.perf_counter()
        relax = sum(pool.map(one, insts))
        dt = time.perf_counter() - t0
        rounds = int(max(1, min(20, budget_s // max(dt, 1e-3))))
        t0 = time.perf_counter()
        relax = sum(sum(pool.map(one, insts)) for _ in range(rounds))
        dt = time.perf_counter() - t0
    return {"value": relax / dt, "unit": "relaxations/s", "cores": cores, **_host_description(), "kind": "port",
            "sample": f"first {n_layers} layers of {len(insts)} cfg3 instances, {rounds} rounds, one thread per instance, "
                      f"{relax:.3g} relaxations in {dt:.2f} s"}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="cfg2", choices=["cfg0", "cfg1", "cfg2", "cfg3", "cfg4", "galvatron_like"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--row-skipping", action="store_true",
                    help="time the library's default (rows that need no arithmetic are filled or left out) instead "
                         "of carrying out every relaxation; the line says so and gives the executed fraction")
    ap.add_argument("--mark-table", action="store_true",
                    help="time the mode that stores the reference's argmin table while relaxing (GDP_KEEP_MARKS) as the "
                         "headline leg (profiling runs of that mode); the line says so")
    ap.add_argument("--headline-only", action="store_true",
                    help="leave out the row-skipping and mark-table legs (profiling runs: the trace then holds the "
                         "headline's launches alone)")
    ap.add_argument("--also", default="cfg3,cfg0,cfg1,cfg4,galvatron_like,sweep_llama_like",
                    help="comma-separated extra workloads summarised in the same line")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run three device-to-device copies of 1 GiB (a kernel of known traffic, to scale the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run) and exit")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs the DP hot path on ONE GPU; --gpus must be 1 "
              "(instances of a batch are independent and would shard by instance with no exchange)", file=sys.stderr)
        return 2

    import ctypes

    from galvatron_dp import _lib
    _lib.lib()                                        # fails loudly when the HIP library is missing
    hip = ctypes.CDLL("libamdhip64.so")               # already mapped by the library above

    def device_sync():
        if hip.hipDeviceSynchronize() != 0:
            raise RuntimeError("hipDeviceSynchronize failed")

    if a.calibrate_copy:
        n = 1 << 30
        src, dst = ctypes.c_void_p(), ctypes.c_void_p()
        assert hip.hipMalloc(ctypes.byref(src), ctypes.c_size_t(n)) == 0
        assert hip.hipMalloc(ctypes.byref(dst), ctypes.c_size_t(n)) == 0
        assert hip.hipMemset(src, 1, ctypes.c_size_t(n)) == 0
        for _ in range(3):
            assert hip.hipMemcpy(dst, src, ctypes.c_size_t(n), 3) == 0      # hipMemcpyDeviceToDevice
        device_sync()
        hip.hipFree(src)
        hip.hipFree(dst)
        print(json.dumps({"calibrate_copy_bytes": n, "copies": 3}))
        return 0

    def measure(workload, steps, warmup, compute_all=True, keep_marks=False, host_leg=False, check=False):
        insts, probs = _problems(workload, compute_all, keep_marks)
        with _lib.Plan(probs) as plan:
            for _ in range(warmup):
                plan.run(0)
            device_sync()
            t0 = time.perf_counter()
            for _ in range(steps):
                plan.run(0)                       # synchronises the plan's stream before returning
            device_sync()
            wall = time.perf_counter() - t0
            tms = sorted((plan.run(2) for _ in range(5)), key=lambda t: t.relax_ms)
            tm = tms[len(tms) // 2]                # per-launch HIP events on the plan's stream: the median of five solves
            t1 = plan.run(1)
            plan.fetch()
        bit_exact = None
        if check:                                  # outside the timed region
            bit_exact = _bit_exact(workload, probs)
            if bit_exact is not None:
                with open(GOLDEN) as fh:
                    golden = json.load(fh)
                names = [f"cfg3_{n:03d}" for n in range(len(insts))] if workload == "cfg3" else [workload]
                bit_exact = bit_exact and all(i.digest() == golden[n]["input_sha256"] for i, n in zip(insts, names))
        # The same solve from host arrays through gdp_solve_batch: validation, layout, upload, all kernels,
        # download (device memory of earlier calls is reused).  Reported beside the headline, never as it.
        host_ms = []
        for _ in range(1 + max(3, min(steps, 5)) if host_leg else 0):
            h0 = time.perf_counter()
            _lib.solve_batch(probs)
            host_ms.append((time.perf_counter() - h0) * 1e3)
        host_ms = sorted(host_ms[1:])[len(host_ms[1:]) // 2] if host_leg else None
        # ... and as ONE call of the drop-in plugin with the reference's eleven arguments (the caller's arrays
        # allocated once, as DPAlg does), for single instances.
        plugin_ms = None
        if host_leg and len(insts) == 1:
            import numpy as np
            import galvatron_dp_core as plugin
            i0 = insts[0]
            res = {k: np.full(i0.L, -1, dtype=np.int32) for k in i0.other_mem}
            inter = np.ascontiguousarray(i0.inter)
            f = np.zeros((i0.V, i0.S))              # DPAlg's ``_f`` (dynamic_programming.py:16); ``_mark`` is never read
            args = (i0.L, i0.V, i0.S, i0.mem, None, f, inter, i0.intra, i0.other_mem, i0.other_time, res)
            times = []
            for _ in range(1 + max(5, min(steps, 30))):
                h0 = time.perf_counter()
                plugin.dynamic_programming_core(*args)
                times.append((time.perf_counter() - h0) * 1e3)
            plugin_ms = sorted(times[1:])[len(times[1:]) // 2]
        relax = tm.relaxations
        launches = tm.relax_launches
        avg_launch_s = tm.relax_ms * 1e-3 / launches
        # fp64 vector operations the kernel issues per relaxation: v_add_f64 + v_min_f64, plus one addition
        # per cell (1/S); with the argmin table two additions, a compare and a minimum (its select is a
        # 32-bit operation, like the two v_readlane per relaxation of the variant for small per-layer
        # launches: not fp64 work, not counted)
        issued = 4.0 if keep_marks else 2.0 + 1.0 / insts[0].S
        per_launch_s = tm.executed / launches / avg_launch_s
        return {
            "insts": insts, "probs": probs, "relaxations": relax, "ms_per_step": wall / steps * 1e3,
            "value": relax * steps / wall, "launches": launches, "avg_launch_ms": avg_launch_s * 1e3,
            "device_ms": t1.total_ms, "host_ms": host_ms, "plugin_ms": plugin_ms, "executed_fraction": tm.executed / relax,
            "tops_issued": issued * per_launch_s / 1e12, "tops_reference": 3.0 * per_launch_s / 1e12,
            "issued_per_relaxation": issued,
            "gbs": tm.relax_bytes / launches / avg_launch_s / 1e9,
            "bytes_per_launch": tm.relax_bytes / launches,
            "scheme": ("fused (all layers in one launch)" if tm.fused else
                       "flow (all layers in one launch, tasks wait on the cost cells themselves)" if tm.flow else
                       "one launch per layer"),
            "tile": "%d target strategies x %d budget rows per wavefront" % (tm.tile_ts, 64 * tm.tile_r),
            "tile_key": "%dx%d" % (tm.tile_ts, tm.tile_r),
            "kernel": "gdp_relax_fused_kernel" if tm.fused else "gdp_relax_flow_kernel" if tm.flow else
                      ("gdp_relax_kernel (latency variant)" if tm.latency_variant else "gdp_relax_kernel"),
            "clock_ghz": PROFILED_CLOCK_GHZ.get(workload) if compute_all and not keep_marks else None,
            "bit_exact": bit_exact,
        }

    def fractions(mm):
        return {"frac": mm["tops_issued"] / PEAK_FP64_VALU_TFLOPS,
                "frac_reference_ops": mm["tops_reference"] / PEAK_FP64_VALU_TFLOPS,
                "frac_hbm": mm["gbs"] / PEAK_HBM_GBS}

    m = measure(a.workload, a.steps, a.warmup, compute_all=not a.row_skipping, keep_marks=a.mark_table,
                host_leg=not a.headline_only, check=True)
    insts = m["insts"]
    first = insts[0]
    traffic, traffic_source = _traffic(a.workload + ("+row_skipping" if a.row_skipping else "") +
                                       ("+mark_table" if a.mark_table else ""), m["tile_key"])
    fr = fractions(m)
    line = {
        "metric": "min-plus relaxations/s (L*V*S^2)", "value": m["value"], "unit": "relaxations/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": m["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f64", "data": "synthetic",
        "config": {"workload": a.workload, "instances": len(insts), "L": first.L if len(insts) == 1 else "32/pp",
                   "S": first.S, "V": first.V, "relaxations_per_step": m["relaxations"],
                   "argmin": ("stored while relaxing (one byte per cell)" if a.mark_table else
                              "recomputed on the backtrack (costs-only relaxation)"),
                   "search_wall_ms_device": m["device_ms"],
                   "search_wall_ms_from_host_arrays": m["host_ms"], "plugin_call_ms": m["plugin_ms"],
                   "launch_scheme": m["scheme"],
                   "register_tile": m["tile"],
                   "relaxations_executed_fraction": m["executed_fraction"], "bit_exact": m["bit_exact"],
                   "device": _lib.device_info()},
        "roofline": {"bound": "valu_fp64", "achieved": m["tops_issued"], "peak": PEAK_FP64_VALU_TFLOPS,
                     "unit": "TFLOP/s", "frac": fr["frac"], "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": m["kernel"], "launches_per_step": m["launches"],
                     "avg_launch_ms": m["avg_launch_ms"],
                     "ops_counted": "fp64 vector operations issued for the relaxations carried out",
                     "issued_ops_per_relaxation": m["issued_per_relaxation"],
                     "frac_reference_ops": fr["frac_reference_ops"], "reference_ops_per_relaxation": 3,
                     "clock_ghz_under_load": m["clock_ghz"], "peak_clock_ghz": 2.4},
        "roofline_hbm": {"bound": "hbm", "achieved": m["gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": fr["frac_hbm"], "traffic": traffic,
                         "algorithmic_bytes_per_launch": m["bytes_per_launch"]},
    }
    also = {}
    for w in [x for x in a.also.split(",") if x and x != a.workload]:
        if w.startswith("sweep_"):
            also[w] = _sweep_leg(w[len("sweep_"):])
            continue
        mm = measure(w, max(3, a.steps // 4), 1, host_leg=not a.headline_only, check=True)
        ff = fractions(mm)
        also[w] = {"value": mm["value"], "ms_per_step": mm["ms_per_step"], "instances": len(mm["insts"]),
                   "search_wall_ms_device": mm["device_ms"],
                   "search_wall_ms_from_host_arrays": mm["host_ms"], "plugin_call_ms": mm["plugin_ms"],
                   "launch_scheme": mm["scheme"], "kernel": mm["kernel"], "register_tile": mm["tile"],
                   "roofline_frac_valu_fp64": ff["frac"], "issued_ops_per_relaxation": mm["issued_per_relaxation"],
                   "roofline_frac_valu_fp64_reference_ops": ff["frac_reference_ops"],
                   "roofline_frac_hbm": ff["frac_hbm"], "avg_launch_ms": mm["avg_launch_ms"],
                   "launches_per_step": mm["launches"], "traffic": _traffic(w, mm["tile_key"])[0],
                   "bit_exact": mm["bit_exact"]}
    if also:
        line["also"] = also
    if a.row_skipping:
        del line["roofline_hbm"]       # its algorithmic bytes are those of the full table
        line["metric"] += " -- NOMINAL count over time with row skipping on; roofline figures count executed relaxations"
    if not a.headline_only:
        # The library's default additionally leaves out rows it can prove irrelevant (all-infinite sources /
        # unreachable from every start row); results are identical, fewer relaxations are carried out.
        ms = measure(a.workload, max(3, a.steps // 2), 1, compute_all=False, check=True)
        line["with_row_skipping"] = {"value_nominal": ms["value"], "ms_per_step": ms["ms_per_step"],
                                     "relaxations_executed_fraction": ms["executed_fraction"],
                                     "roofline_frac_valu_fp64_executed": fractions(ms)["frac"],
                                     "bit_exact": ms["bit_exact"]}
        mk = measure(a.workload, max(3, a.steps // 2), 1, keep_marks=True, check=True)
        line["with_mark_table"] = {"value": mk["value"], "ms_per_step": mk["ms_per_step"],
                                   "issued_ops_per_relaxation": mk["issued_per_relaxation"],
                                   "roofline_frac_valu_fp64": fractions(mk)["frac"],
                                   "roofline_frac_valu_fp64_reference_ops": fractions(mk)["frac_reference_ops"],
                                   "algorithmic_bytes_per_launch": mk["bytes_per_launch"],
                                   "bit_exact": mk["bit_exact"]}
    if not a.no_cpu_baseline:
        line["cpu_baseline"] = _cpu_baseline(a.workload)
        line["vs_cpu_baseline_same_run"] = {
            "ratio": m["value"] / line["cpu_baseline"]["value"],
            "meaning": "value / cpu_baseline.value: the same-run figure of the reference's code on one core of this "
                       "host, not a published baseline (vs_baseline stays null: none is published)"}
        if "cfg3" in also:
            also["cfg3"]["cpu_baseline_all_cores"] = _cpu_baseline_all_cores()
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
