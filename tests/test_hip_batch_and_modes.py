"""GPU tests of the batched entry points and of the two launch schemes (one launch per layer /
one launch for all layers), through the C ABI."""
import os

import numpy as np
import pytest

import helpers as H
from galvatron_dp import _lib, workloads as W

pytestmark = pytest.mark.gpu


def _problem(inst, **kw):
    keys = sorted(inst.other_mem)
    return _lib.Problem(inst.mem, inst.intra, inst.inter_tables, inst.V, [inst.other_mem[k] for k in keys],
                        [inst.other_time[k] for k in keys], inter_index=inst.inter_index, **kw)


def _check_against_golden(prob, rec, name):
    keys = rec["keys"]
    got = ({k: prob.total[i] for i, k in enumerate(keys)},
           {k: [int(x) if prob.remaining[i] != -1 else -1 for x in prob.res[i]] for i, k in enumerate(keys)},
           {k: int(prob.remaining[i]) for i, k in enumerate(keys)})
    H.assert_same_results(got, H.golden_results(rec), name)


def test_batched_sweep_256_instances_matches_reference(golden):
    """Workload cfg3: all 256 instances of the pp x bsz x chunks sweep in ONE gdp_solve_batch
    call, every instance compared with the reference's result for it."""
    insts = W.config3()
    assert len(insts) == 256
    probs = [_problem(i) for i in insts]
    _lib.solve_batch(probs)
    for n, (inst, prob) in enumerate(zip(insts, probs)):
        rec = golden[f"cfg3_{n:03d}"]
        assert inst.digest() == rec["input_sha256"]
        _check_against_golden(prob, rec, f"cfg3_{n:03d}")


def test_mixed_shapes_in_one_batch(golden):
    """Instances with different L, S and V in one call (grouped by S internally) come back in the
    caller's order."""
    names = ["ties_1", "rand_2", "cfg3_smallV_0", "infeasible_3", "rand_5", "cfg3_smallV_3", "ties_6", "rand_7",
             "cfg2_small", "rand_8", "cfg4_small", "galvatron_like"]
    insts = [H.build_case(golden[n]) for n in names]
    probs = [_problem(i) for i in insts]
    _lib.solve_batch(probs)
    for n, prob in zip(names, probs):
        _check_against_golden(prob, golden[n], n)


@pytest.mark.parametrize("fused", [0, 1])
@pytest.mark.parametrize("name", ["cfg2_small", "cfg4_small", "galvatron_like", "ties_6", "infeasible_9"])
def test_both_launch_schemes_give_identical_arrays(golden, name, fused):
    rec = golden[name]
    inst = H.build_case(rec)
    prob = _problem(inst, export_f=True, export_mark=True, launch="fused" if fused else "per_layer")
    with _lib.Plan([prob]) as plan:
        plan.set_option(_lib.GDP_OPT_POISON, 1)       # unwritten cells read as NaN: a stale read would show
        for _ in range(2):                             # a plan can be run again and again
            plan.run()
            plan.fetch()
            _check_against_golden(prob, rec, name)
            assert H.sha(prob.f_out) == rec["f_sha256"]
            assert H.sha(prob.mark_out) == rec["mark_sha256"]


@pytest.mark.parametrize("launch", ["fused", "per_layer"])
@pytest.mark.parametrize("name", ["cfg2_small", "cfg4_small", "galvatron_like", "infeasible_6", "cfg3_smallV_5"])
def test_skipping_rows_changes_nothing(golden, name, launch):
    """Rows whose sources are all +inf are filled, rows no start row can reach back to are left out:
    same results as computing every cell, and fewer relaxations carried out."""
    rec = golden[name]
    inst = H.build_case(rec)
    done = {}
    for compute_all in (True, False):
        prob = _problem(inst, launch=launch, compute_all=compute_all)
        with _lib.Plan([prob]) as plan:
            plan.set_option(_lib.GDP_OPT_POISON, 1)
            t = plan.run(1)
            plan.fetch()
        _check_against_golden(prob, rec, f"{name} compute_all={compute_all}")
        done[compute_all] = t.executed / t.relaxations
    assert abs(done[True] - 1.0) < 1e-12 and done[False] <= 1.0
    # with the full arrays requested only the +inf rows may be skipped, and the arrays stay identical
    prob = _problem(inst, launch=launch, export_f=True, export_mark=True)
    _lib.solve_batch([prob])
    assert H.sha(prob.f_out) == rec["f_sha256"] and H.sha(prob.mark_out) == rec["mark_sha256"]


@pytest.mark.parametrize("launch", ["fused", "per_layer"])
@pytest.mark.parametrize("keep_marks", [False, True])
@pytest.mark.parametrize("name", ["cfg2_small", "cfg4_small", "galvatron_like", "ties_3", "infeasible_6",
                                  "cfg3_smallV_2"])
def test_costs_only_and_mark_table_modes_agree(golden, name, launch, keep_marks):
    """Default: the relaxation stores costs only and the backtrack recomputes the argmin of the cells
    on its path.  keep_marks: the argmin table is stored as in the reference.  Same results, same f."""
    rec = golden[name]
    inst = H.build_case(rec)
    prob = _problem(inst, launch=launch, keep_marks=keep_marks, export_f=True)
    with _lib.Plan([prob]) as plan:
        plan.set_option(_lib.GDP_OPT_POISON, 1)
        t = plan.run(1)
        plan.fetch()
    _check_against_golden(prob, rec, f"{name} keep_marks={keep_marks}")
    assert H.sha(prob.f_out) == rec["f_sha256"]
    if "GALVATRON_DP_KEEP_MARKS" not in os.environ:     # a preset in the environment overrides the flag
        cells = float(inst.L) * inst.V * inst.S
        assert t.relax_bytes == cells * (17 if keep_marks else 16)


@pytest.mark.parametrize("keep_marks", [False, True])
@pytest.mark.parametrize("name", [f"zeromem_{i}" for i in range(8)])
def test_memory_costs_of_zero_with_rows_skipped_and_unwritten_cells_poisoned(golden, name, keep_marks):
    """The pass that redoes the strategies with a memory cost of 0 keeps to the layer's band: rows above
    it were never written by the layer's launch (they read as NaN here), rows below it hold their fill."""
    rec = golden[name]
    inst = H.build_case(rec)
    prob = _problem(inst, keep_marks=keep_marks)
    with _lib.Plan([prob]) as plan:
        plan.set_option(_lib.GDP_OPT_POISON, 1)
        for run in range(2):
            t = plan.run(1)
            plan.fetch()
            _check_against_golden(prob, rec, f"{name} keep_marks={keep_marks} run {run}")
    assert t.executed <= t.relaxations


def test_batch_solved_in_parts_and_allocation_reuse(golden, monkeypatch):
    """A batch above the device-memory budget of one allocation is solved in consecutive parts; the
    allocation of a finished plan is reused by the next one (stale contents must not matter) and
    can be given back."""
    names = ["cfg3_smallV_%d" % i for i in range(8)] + ["ties_2", "cfg2_small", "infeasible_4"]
    insts = [H.build_case(golden[n]) for n in names]
    monkeypatch.setenv("GALVATRON_DP_ARENA_MB", "1")        # every instance becomes a part of its own
    for rep in range(2):
        probs = [_problem(i) for i in insts]
        _lib.solve_batch(probs)
        for n, prob in zip(names, probs):
            _check_against_golden(prob, golden[n], f"{n} rep {rep}")
    monkeypatch.setenv("GALVATRON_DP_CACHE_MB", "0")        # nothing is kept from here on
    probs = [_problem(i) for i in insts]
    _lib.solve_batch(probs)
    for n, prob in zip(names, probs):
        _check_against_golden(prob, golden[n], n)
    _lib.cache_trim()
    monkeypatch.delenv("GALVATRON_DP_ARENA_MB")
    probs = [_problem(i) for i in insts]
    _lib.solve_batch(probs)
    for n, prob in zip(names, probs):
        _check_against_golden(prob, golden[n], n)


def test_streams_and_result_buffers_handed_from_plan_to_plan(golden):
    """A finished plan leaves its stream and page-locked result buffer to the next plan.  Plans whose
    results are smaller, then larger than the buffer they inherit, plans alive at the same time (each
    needs a set of its own), fetch after a later plan has run, and giving everything back in between."""
    small = ["ties_2", "infeasible_2", "rand_2"]
    big = ["cfg3_smallV_%d" % i for i in range(8)] * 40          # 320 instances: > 64 KB of results
    for rep in range(3):
        for names in (small, big, small[:1]):
            probs = [_problem(H.build_case(golden[n])) for n in names]
            _lib.solve_batch(probs)
            for n, prob in zip(names, probs):
                _check_against_golden(prob, golden[n], f"{n} rep {rep}")
        if rep == 1:
            _lib.cache_trim()
    pa = [_problem(H.build_case(golden[n])) for n in small]
    pb = [_problem(H.build_case(golden[n])) for n in big[:8]]
    with _lib.Plan(pa) as a, _lib.Plan(pb) as b:
        a.run()
        b.run()
        b.run()
        a.fetch()               # a's results were copied back by a's own run, into a's own buffer
        b.fetch()
    for n, prob in zip(small + big[:8], pa + pb):
        _check_against_golden(prob, golden[n], n)


@pytest.mark.parametrize("S", [1, 7, 8, 9, 15, 16, 17, 40, 44, 63, 100])
def test_small_launches_use_the_latency_variant(S, monkeypatch):
    """One small instance, one launch per layer: the narrowest tile runs in the variant that keeps
    scalar loads out of its loop (sources padded to 8 per trip, transition costs spread from a vector
    register), the sources of a task on 1, 2 or 4 waves whose partial minima meet in LDS.  Same bits
    as the ordinary variant and as the oracle, f included; S on both sides of the trip length and of
    the tile width."""
    if any(k in os.environ for k in ("GALVATRON_DP_KEEP_MARKS", "GALVATRON_DP_TILE_TS", "GALVATRON_DP_TILE_R",
                                     "GALVATRON_DP_FUSED", "GALVATRON_DP_LATENCY_VARIANT")):
        pytest.skip("the environment presets the layout")
    from oracle import dp_oracle as O
    monkeypatch.setenv("GALVATRON_DP_FLOW", "0")     # (a plan this small would otherwise run all layers in one flow launch)
    rng = np.random.Generator(np.random.PCG64([3, S]))
    inst = W.random_instance(rng, 5, S, 700 + S, mem_hi=150, inf_frac=0.1, per_layer_inter=bool(S % 2), n_keys=3)
    wt, wr, wm, wf, _ = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time, keep=True)
    keys = sorted(inst.other_mem)
    seen = []
    for preset in (None, "0", "1", "2", "4"):
        if preset is not None:
            monkeypatch.setenv("GALVATRON_DP_LATENCY_VARIANT", preset)
        prob = _problem(inst, export_f=True)
        with _lib.Plan([prob]) as plan:
            plan.set_option(_lib.GDP_OPT_POISON, 1)
            t = plan.run(1)
            plan.fetch()
        seen.append((t.fused, t.tile_ts, t.tile_r, t.latency_variant))
        got = ({k: prob.total[i] for i, k in enumerate(keys)}, {k: [int(x) for x in prob.res[i]] for i, k in enumerate(keys)},
               {k: int(prob.remaining[i]) for i, k in enumerate(keys)})
        H.assert_same_results(got, (wt, wr, wm), f"S={S} preset={preset}")
        assert prob.f_out.tobytes() == wf.tobytes()
    assert seen[0] == (0, 8, 1, 4 if S >= 32 else 1)        # 12..13 tiles: room for four waves per task
    assert seen[1:] == [(0, 8, 1, 0), (0, 8, 1, 1), (0, 8, 1, 2), (0, 8, 1, 4)]


def test_fused_runs_from_several_threads_take_turns(golden):
    """Workgroups of a fused launch wait for earlier ones of the same launch; two such launches side
    by side could each fill XCDs that the other needs.  The library lets one fused launch run at a
    time, so none of them ever has to give up (which would take seconds), whatever the threads do."""
    import threading
    if os.environ.get("GALVATRON_DP_FUSED") == "0":
        pytest.skip("the environment presets per-layer launches")
    names = ["cfg3_smallV_%d" % i for i in range(8)] * 12         # 96 instances: enough blocks to fill the device
    errors, gave_up = [], []

    def work(k):
        try:
            probs = [_problem(H.build_case(golden[n]), launch="fused") for n in names]
            with _lib.Plan(probs) as plan:
                plan.set_option(_lib.GDP_OPT_NO_FALLBACK, 1)   # an abandoned launch raises instead of switching
                for _ in range(6):
                    t = plan.run(1)
                    gave_up.append(not t.fused)
                plan.fetch()
            for n, prob in zip(names, probs):
                _check_against_golden(prob, golden[n], f"thread {k} {n}")
        except Exception as e:  # noqa: BLE001
            errors.append((k, repr(e)))

    threads = [threading.Thread(target=work, args=(k,)) for k in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert not any(gave_up)     # (no bound on the wall time: a shared box may be slow and still be right)


@pytest.mark.parametrize("chunk,max_rows", [(1, 65535), (3, 65535), (2, 5), (1000, 3), (4, 1)])
def test_instances_taken_through_the_launch_a_few_at_a_time(golden, monkeypatch, chunk, max_rows):
    """A fused launch takes `chunk` instances at a time through all their layers (grid rows follow a
    table; more rows than a grid holds are split over launches -- forced here with a tiny limit).
    Mixed depths, widths and budgets in one batch; chunk sizes that do and do not divide the groups."""
    names = ["cfg3_smallV_%d" % i for i in range(8)] + ["ties_6", "rand_6", "infeasible_6", "ties_2", "cfg2_small",
                                                        "rand_2", "infeasible_2"]
    insts = [H.build_case(golden[n]) for n in names]
    monkeypatch.setenv("GALVATRON_DP_CHUNK", str(chunk))
    monkeypatch.setenv("GALVATRON_DP_MAX_GRID_ROWS", str(max_rows))
    probs = [_problem(i, launch="fused") for i in insts]
    with _lib.Plan(probs) as plan:
        plan.set_option(_lib.GDP_OPT_POISON, 1)
        for _ in range(2):
            t = plan.run(1)
            plan.fetch()
            for n, prob in zip(names, probs):
                _check_against_golden(prob, golden[n], f"{n} chunk={chunk} rows={max_rows}")
    if "GALVATRON_DP_FUSED" not in os.environ:          # a preset in the environment overrides the flag
        assert t.fused
        if max_rows < 10:
            assert t.relax_launches > 4


def test_plan_reports_its_layout(golden):
    """The register tile follows the documented rule: fewest target blocks that still fill the device
    (costs only), least padding with the argmin table; the timing record says what was chosen."""
    if any(k in os.environ for k in ("GALVATRON_DP_KEEP_MARKS", "GALVATRON_DP_TILE_TS", "GALVATRON_DP_TILE_R")):
        pytest.skip("the environment presets the layout")

    def layout(insts, **kw):
        with _lib.Plan([_problem(i, **kw) for i in insts]) as plan:
            t = plan.run(1)
        return t.tile_ts, t.keep_marks

    small64 = H.build_case(golden["cfg2_small"])                # one instance, S = 64, V = 12288: under-filled
    assert layout([small64]) == (8, 0)                          # the most blocks there are
    assert layout([small64] * 24) == (16, 0)                    # enough work: four blocks of 16
    assert layout([small64] * 24, keep_marks=True) == (8, 1)    # argmin table: least padding among 8 / 11
    s44 = [H.build_case(golden["cfg3_smallV_%d" % i]) for i in range(8)]   # S = 44, V = 8192
    assert layout(s44 * 8) == (15, 0)                           # three blocks of 15
    assert layout(s44 * 8, keep_marks=True) == (11, 1)
    assert layout([H.build_case(golden["cfg4_small"])] * 16)[0] == 15      # S = 88: six blocks of 15


def test_device_memory_short_for_one_buffer_per_layer(golden, monkeypatch):
    """A device too full for one cost buffer per layer: plan creation starts over with two cost
    buffers and the argmin table (and the register tiles that exist for that mode; S = 64 uses a
    16-wide tile otherwise), with the same results; too full for that as well: MemoryError.  The
    shortage is forced from the host (allocation requests above a limit are refused)."""
    rec = golden["cfg2_small"]                         # L=12, S=64, V=12288: ~90 MB against ~25 MB
    inst = H.build_case(rec)
    _lib.cache_trim()
    monkeypatch.setenv("GALVATRON_DP_DEVICE_LIMIT_MB", "48")
    prob = _problem(inst, export_f=True)
    with _lib.Plan([prob]) as plan:
        t = plan.run(1)
        plan.fetch()
    _check_against_golden(prob, rec, "cfg2_small under a 48 MB limit")
    assert H.sha(prob.f_out) == rec["f_sha256"]
    assert t.relax_bytes == float(inst.L) * inst.V * inst.S * 17 and not t.fused
    monkeypatch.setenv("GALVATRON_DP_DEVICE_LIMIT_MB", "4")
    with pytest.raises(MemoryError):
        _lib.solve_batch([_problem(inst)])
    monkeypatch.delenv("GALVATRON_DP_DEVICE_LIMIT_MB")
    prob = _problem(inst)
    _lib.solve_batch([prob])
    _check_against_golden(prob, rec, "cfg2_small afterwards")


def test_abandoned_fused_launch_falls_back_or_reports(golden):
    """A spin limit of 1 makes waiting wavefronts give up at once (forced from the host; every
    kernel still runs to completion).  With the fallback the plan switches to per-layer launches
    and returns the right answer; without it the run reports an error.  Either way the next call
    on a fresh plan works."""
    rec = golden["cfg2_small"]
    inst = H.build_case(rec)
    prob = _problem(inst, launch="fused")
    with _lib.Plan([prob]) as plan:
        plan.set_option(_lib.GDP_OPT_SPIN_LIMIT, 1)
        plan.run()
        plan.fetch()
        _check_against_golden(prob, rec, "fallback")
    prob2 = _problem(inst, launch="fused")
    with _lib.Plan([prob2]) as plan:
        plan.set_option(_lib.GDP_OPT_SPIN_LIMIT, 1)
        plan.set_option(_lib.GDP_OPT_NO_FALLBACK, 1)
        try:
            plan.run()
            gave_up = False
        except RuntimeError as e:
            gave_up = True
            assert "bounded wait" in str(e)
        if not gave_up:                               # every wait happened to be satisfied at its first poll
            plan.fetch()
            _check_against_golden(prob2, rec, "no-fallback, nothing had to wait")
    prob3 = _problem(inst)
    _lib.solve_batch([prob3])
    _check_against_golden(prob3, rec, "after")


def test_a_wait_that_cannot_end_costs_milliseconds_and_the_plan_is_armed_again(golden, monkeypatch):
    """The first layer of the fused launch leaves its completion counters alone (forced from the host; every
    kernel still ends normally), so the waits of the second layer run into their bound.  That bound follows
    from the plan's size -- 5 ms for a plan this small, where a fixed number of polls used to take a second --
    after which the solve is repeated with one launch per layer and gives the right answer.  Once the time has
    passed for which the library avoids waiting launches, the plan runs with its own launch scheme again."""
    import time
    rec = golden["cfg2_small"]
    inst = H.build_case(rec)
    monkeypatch.setenv("GALVATRON_DP_SHARED_BACKOFF_MS", "150")
    prob = _problem(inst, launch="fused")
    try:
        with _lib.Plan([prob]) as plan:
            assert plan.run(1).fused == 1
            plan.set_option(_lib.GDP_OPT_DEBUG_STALL, 1)
            t0 = time.perf_counter()
            t = plan.run(1)
            dt = time.perf_counter() - t0
            plan.fetch()
            _check_against_golden(prob, rec, "after the bounded wait ran out")
            assert t.fused == 0 and t.relax_launches == inst.L
            assert dt < 0.25, f"give-up and repeated solve took {dt * 1e3:.0f} ms"
            plan.set_option(_lib.GDP_OPT_DEBUG_STALL, 0)
            assert plan.run(1).fused == 0                  # still inside the back-off: one launch per layer
            time.sleep(0.3)
            t = plan.run(1)
            plan.fetch()
            assert t.fused == 1, "the plan was not armed again after the back-off"
            _check_against_golden(prob, rec, "armed again")
    finally:
        _lib.debug_shared_device(False)


def test_shim_batch_entry_point(golden):
    import galvatron_dp_core as shim
    names = ["rand_1", "ties_3", "infeasible_5"]
    calls, want = [], []
    for n in names:
        inst = H.build_case(golden[n])
        res = {k: np.full(inst.L, -1, dtype=np.int32) for k in inst.other_mem}
        calls.append((inst.L, inst.V, inst.S, inst.mem, None, None, inst.inter, inst.intra, inst.other_mem,
                      inst.other_time, res))
        want.append(golden[n])
    outs = shim.dynamic_programming_core_batch(calls)
    for (total, rem), call, rec, n in zip(outs, calls, want, names):
        got = (total, {k: [int(x) for x in v] for k, v in call[10].items()}, rem)
        H.assert_same_results(got, H.golden_results(rec), n)


def test_errors_surface_as_python_exceptions():
    import galvatron_dp_core as shim
    L, S, V = 2, 3, 16
    mem = np.ones((L, S), np.int32)
    intra = np.ones((L, S))
    inter = np.zeros((L, S, S))
    res = {1: np.full(L, -1, np.int32)}
    bad = mem.copy(); bad[0, 0] = -1
    with pytest.raises(ValueError):
        shim.dynamic_programming_core(L, V, S, bad, None, None, inter, intra, {1: 0}, {1: 0.0}, res)
    with pytest.raises(ValueError):                       # start row above the table
        shim.dynamic_programming_core(L, V, S, mem, None, None, inter, intra, {1: -3}, {1: 0.0}, res)
    nan = intra.copy(); nan[1, 1] = np.nan
    with pytest.raises(ValueError):
        shim.dynamic_programming_core(L, V, S, mem, None, None, inter, nan, {1: 0}, {1: 0.0}, res)
    total, rem = shim.dynamic_programming_core(L, V, S, mem, None, None, inter, intra, {1: 0, 2: 99}, {1: 0.5, 2: 0.0},
                                               {1: res[1], 2: np.full(L, -1, np.int32)})
    assert total == {1: 2.5, 2: np.inf} and rem == {1: V - 1 - 2, 2: -1} and list(res[1]) == [0, 0]
