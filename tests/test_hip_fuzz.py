"""Differential test on the GPU: seeded random instances through the plugin signature against
the C oracle, on shapes chosen to hit the kernel's corners: S around the register-tile widths
(8, 11) and the wavefront width (63..65, 127..129, 255..257, 300, 513, 1000, 1024 = the largest), V not a multiple of any tile height,
memory costs near 1, near V and above V, +inf costs, exact ties, shared and per-layer inter
matrices, start rows below 0.  Full f and mark arrays are compared as well as the results."""
import os

import numpy as np
import pytest

import helpers as H
from galvatron_dp import _lib, workloads as W
from oracle import dp_oracle as O

pytestmark = pytest.mark.gpu

SHAPES = [(1, 1, 1), (1, 1, 7), (2, 1, 64), (3, 2, 65), (4, 7, 191), (3, 8, 192), (5, 9, 193), (2, 10, 255),
          (6, 11, 256), (3, 12, 257), (4, 16, 383), (2, 21, 385), (7, 22, 512), (3, 23, 700), (2, 33, 129),
          (3, 44, 1000), (2, 45, 130), (2, 63, 300), (3, 64, 333), (2, 65, 200), (2, 88, 410), (1, 127, 150),
          (2, 128, 140), (2, 129, 131), (1, 255, 90), (2, 256, 70), (9, 5, 2048), (12, 3, 4099), (20, 4, 1500),
          (2, 257, 70), (2, 300, 150), (1, 513, 40), (3, 13, 200), (3, 14, 333), (2, 26, 300), (2, 28, 129),
          (2, 39, 150), (2, 42, 200), (2, 52, 140), (2, 56, 190), (2, 60, 130), (2, 74, 100), (1, 1000, 33),
          (1, 1024, 30)]


def _compare(inst, tag, launch=None):
    """Two solves of the same instance: costs-only relaxation with the argmin recomputed on the
    backtrack (the default; f exported, which does not change the mode) and the mode that keeps
    the reference's mark table (forced by exporting it)."""
    keys = sorted(inst.other_mem)
    wt, wr, wm, wf, wmark = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time,
                                    keep=True)
    for marks in ((False, True) if inst.S <= _lib.GDP_MAX_S_MARKS else (False,)):   # mark entries are bytes
        prob = _lib.Problem(inst.mem, inst.intra, inst.inter_tables, inst.V, [inst.other_mem[k] for k in keys],
                            [inst.other_time[k] for k in keys], inter_index=inst.inter_index, export_f=True,
                            export_mark=marks, launch=launch)
        with _lib.Plan([prob]) as plan:
            plan.set_option(_lib.GDP_OPT_POISON, 1)
            plan.run()
            plan.fetch()
        got = ({k: prob.total[i] for i, k in enumerate(keys)},
               {k: [int(x) for x in prob.res[i]] for i, k in enumerate(keys)},
               {k: int(prob.remaining[i]) for i, k in enumerate(keys)})
        H.assert_same_results(got, (wt, wr, wm), f"{tag} marks={marks}")
        assert prob.f_out.tobytes() == wf.tobytes(), f"{tag} marks={marks}: f differs"
        if marks:
            assert np.array_equal(prob.mark_out, wmark), f"{tag}: mark differs"


@pytest.mark.parametrize("n,shape", list(enumerate(SHAPES)))
def test_random_instances_against_oracle(n, shape, monkeypatch):
    L, S, V = shape
    if S > _lib.GDP_MAX_S_MARKS and os.environ.get("GALVATRON_DP_KEEP_MARKS", "0") != "0":
        pytest.skip("the environment forces the argmin table, whose entries are bytes")
    for variant in range(4):
        rng = np.random.Generator(np.random.PCG64([77, n, variant]))
        ties = variant in (1, 3)
        hi = [max(1, V // (L + 1)), max(1, V // 2), V + 3, 3][variant]
        inst = W.random_instance(rng, L, S, V, integer_costs=ties, mem_hi=hi, per_layer_inter=bool(variant % 2),
                                 inf_frac=0.2 if variant >= 2 else 0.0, over_frac=0.1 if variant == 3 else 0.0,
                                 n_keys=min(4, 1 + variant))
        # small per-layer launches use a kernel variant of their own; variant 2 runs without it
        if variant == 2 and "GALVATRON_DP_LATENCY_VARIANT" not in os.environ:
            monkeypatch.setenv("GALVATRON_DP_LATENCY_VARIANT", "0")
        _compare(inst, f"shape {shape} variant {variant}", launch=("fused", "per_layer", None, None)[variant])
        if variant == 2:
            monkeypatch.undo()


ZERO_SHAPES = [(1, 1, 1), (3, 2, 9), (4, 7, 191), (5, 9, 193), (6, 11, 256), (3, 16, 383), (4, 22, 512), (3, 44, 1000),
               (2, 64, 333), (2, 65, 200), (2, 88, 410), (2, 129, 131), (9, 5, 2048), (2, 257, 70), (1, 1024, 30)]


@pytest.mark.parametrize("n,shape", list(enumerate(ZERO_SHAPES)))
def test_memory_costs_of_zero_follow_the_in_place_order(n, shape):
    """A strategy with mem == 0 reads its own row, where lower strategies already hold the layer's values
    (csrc/dp_core.cpp:58-73; the oracle updates in place exactly like the reference).  All-zero layers,
    zeros among ordinary costs, ties, +inf costs, single zero columns; whatever launch scheme is asked
    for, costs-only and with the argmin table, full f and mark arrays compared."""
    L, S, V = shape
    if S > _lib.GDP_MAX_S_MARKS and os.environ.get("GALVATRON_DP_KEEP_MARKS", "0") != "0":
        pytest.skip("the environment forces the argmin table, whose entries are bytes")
    for variant in range(4):
        rng = np.random.Generator(np.random.PCG64([91, n, variant]))
        hi = [0, 1, 3, max(1, V // (L + 1))][variant]
        inst = W.random_instance(rng, L, S, V, mem_lo=0, mem_hi=hi, integer_costs=variant in (1, 3),
                                 per_layer_inter=bool(variant % 2), inf_frac=0.15 if variant >= 2 else 0.0,
                                 over_frac=0.1 if variant == 3 else 0.0, n_keys=min(4, 1 + variant))
        if variant == 3:                                  # mostly ordinary costs, a sprinkling of zeros
            inst.mem[(inst.mem == 0) & (rng.uniform(size=inst.mem.shape) < 0.7)] = max(1, V // (2 * L + 2))
            inst.mem[rng.integers(0, L), rng.integers(0, S)] = 0
        assert (inst.mem == 0).any()
        _compare(inst, f"zero shape {shape} variant {variant}", launch=("fused", "per_layer", None, None)[variant])


@pytest.mark.parametrize("shape", [(4, 8, 300), (3, 16, 200), (5, 11, 257), (3, 64, 150), (2, 44, 129)])
def test_candidates_that_collide_only_after_the_intra_addition(shape, monkeypatch):
    """Transition costs that differ in the last bits under intra costs some 2^40 times larger: many
    candidates (f + inter) + intra are then EQUAL although their (f + inter) differ, so the reference's
    lowest-index rule picks a source that is not the one with the smallest f + inter.  The costs-only
    relaxation takes the minimum before adding intra (the cost is the same, rounding being monotone);
    the strategies must still be the reference's, in both modes and both launch schemes."""
    L, S, V = shape
    rng = np.random.Generator(np.random.PCG64([91, L, S, V]))
    inst = W.random_instance(rng, L, S, V, mem_hi=max(1, V // (L + 1)), per_layer_inter=True, n_keys=3)
    inst.inter_tables[...] = 1.0 + rng.integers(0, 6, size=inst.inter_tables.shape) * 2.0 ** -50
    inst.inter[...] = inst.inter_tables[inst.inter_index]
    inst.intra[...] = 2.0 ** 20 * rng.integers(1, 4, size=inst.intra.shape)
    wt, wr, wm, wf, wmark = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time, keep=True)
    # the scenario does what it is meant to: some cell's reference argmin is not its argmin of f + inter
    f0 = np.zeros((V, S))
    differs = 0
    for v in range(V):
        for s in range(S):
            if v >= inst.mem[0][s]:
                pre = f0[v - inst.mem[0][s]] + inst.inter[0][:, s]
                differs += int(np.argmin(pre)) != int(wmark[0][v][s])
    assert differs > 0
    for launch in ("fused", "per_layer"):
        _compare(inst, f"collisions {shape} {launch}", launch=launch)
    if "GALVATRON_DP_LATENCY_VARIANT" not in os.environ:
        monkeypatch.setenv("GALVATRON_DP_LATENCY_VARIANT", "0")    # the ordinary variant of the narrowest tile
        _compare(inst, f"collisions {shape} per_layer, ordinary variant", launch="per_layer")


def test_no_keys_and_single_layer():
    rng = np.random.Generator(np.random.PCG64(5))
    inst = W.random_instance(rng, 1, 6, 50, mem_hi=20)
    prob = _lib.Problem(inst.mem, inst.intra, inst.inter, 50, [], [], export_f=True)
    _lib.solve_batch([prob])
    wf = O.solve(inst.mem, inst.intra, inst.inter, 50, {}, {}, keep=True)[3]
    assert prob.f_out.tobytes() == wf.tobytes()


def test_start_row_outside_the_table():
    rng = np.random.Generator(np.random.PCG64(6))
    inst = W.random_instance(rng, 3, 4, 40, mem_hi=5)
    inst.other_mem = {1: 0, 2: 39, 3: 40, 4: 10 ** 9}
    inst.other_time = {k: 1.0 for k in inst.other_mem}
    _compare(inst, "start rows 39, -1, far below 0")


def test_many_threads_share_the_library():
    """ctypes releases the GIL; concurrent calls from several threads must not disturb each other."""
    import threading
    rng = np.random.Generator(np.random.PCG64(8))
    insts = [W.random_instance(rng, 4 + i % 3, 10 + i, 600 + 37 * i, mem_hi=60) for i in range(12)]
    want = [O.solve(i.mem, i.intra, i.inter, i.V, i.other_mem, i.other_time) for i in insts]
    errors = []

    def work(k):
        try:
            for _ in range(3):
                got = H.hip_solve(insts[k])
                H.assert_same_results(got, want[k], f"thread {k}")
        except Exception as e:  # noqa: BLE001
            errors.append((k, repr(e)))

    threads = [threading.Thread(target=work, args=(k,)) for k in range(len(insts))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


SPLIT_SHAPES = [(3, 1, 64), (4, 7, 191), (5, 11, 256), (3, 12, 257), (4, 22, 512), (3, 33, 700), (6, 44, 1000), (2, 45, 130),
                (3, 64, 333), (2, 88, 410), (2, 129, 131), (9, 23, 2048), (12, 44, 4099), (2, 300, 150)]


@pytest.mark.parametrize("n,shape", list(enumerate(SPLIT_SHAPES)))
def test_sources_of_a_task_split_over_two_waves(n, shape, monkeypatch):
    """Fused launches whose layers hold few wave tasks put the source strategies of a task on two waves
    (partial minima combined through LDS: exact, the minimum being associative).  Forced here on every shape
    -- odd numbers of sources, fewer sources than a trip, rows that do not fill a tile, +inf, ties -- with
    unwritten cells poisoned, against the C oracle: results and the full f array."""
    if any(k in os.environ for k in ("GALVATRON_DP_KEEP_MARKS", "GALVATRON_DP_TILE_TS", "GALVATRON_DP_TILE_R",
                                     "GALVATRON_DP_FUSED", "GALVATRON_DP_SPLIT")):
        pytest.skip("the environment presets the layout")
    L, S, V = shape
    monkeypatch.setenv("GALVATRON_DP_TILE_TS", "11")
    monkeypatch.setenv("GALVATRON_DP_TILE_R", "1")
    monkeypatch.setenv("GALVATRON_DP_SPLIT", "2")
    for variant in range(3):
        rng = np.random.Generator(np.random.PCG64([78, n, variant]))
        inst = W.random_instance(rng, L, S, V, integer_costs=variant == 1, mem_hi=[max(1, V // (L + 1)), max(1, V // 2), V + 3][variant],
                                 per_layer_inter=bool(variant % 2), inf_frac=0.2 if variant == 2 else 0.0,
                                 over_frac=0.1 if variant == 2 else 0.0, n_keys=3)
        keys = sorted(inst.other_mem)
        want = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time, keep=True)
        for compute_all in (False, True):
            prob = _lib.Problem(inst.mem, inst.intra, inst.inter_tables, inst.V, [inst.other_mem[k] for k in keys],
                                [inst.other_time[k] for k in keys], inter_index=inst.inter_index, export_f=compute_all,
                                launch="fused", compute_all=compute_all)
            with _lib.Plan([prob]) as plan:
                plan.set_option(_lib.GDP_OPT_POISON, 1)
                for _ in range(2):
                    t = plan.run(1)
                    assert t.fused == 1 and t.fused_split == 2 and t.tile_ts == 11 and t.tile_r == 1
                    plan.fetch()
                    got = ({k: prob.total[i] for i, k in enumerate(keys)},
                           {k: [int(x) for x in prob.res[i]] for i, k in enumerate(keys)},
                           {k: int(prob.remaining[i]) for i, k in enumerate(keys)})
                    H.assert_same_results(got, want[:3], f"split, shape {shape} variant {variant} compute_all={compute_all}")
                    if compute_all:
                        assert prob.f_out.tobytes() == want[3].tobytes()
            # the same plan given up (host-forced) repeats the solve with one launch per layer, tasks whole again
            with _lib.Plan([prob]) as plan:
                plan.set_option(_lib.GDP_OPT_SPIN_LIMIT, 1)
                plan.run()
                plan.fetch()
                got = ({k: prob.total[i] for i, k in enumerate(keys)},
                       {k: [int(x) for x in prob.res[i]] for i, k in enumerate(keys)},
                       {k: int(prob.remaining[i]) for i, k in enumerate(keys)})
                H.assert_same_results(got, want[:3], f"split plan after a give-up, shape {shape} variant {variant}")


def test_split_tasks_in_a_batch_of_different_depths(monkeypatch):
    """Several instances of one strategy count, different depths and budgets, in one plan whose fused
    launches split their tasks' sources (one launch per run of layers with the same set of instances)."""
    if any(k in os.environ for k in ("GALVATRON_DP_KEEP_MARKS", "GALVATRON_DP_TILE_TS", "GALVATRON_DP_TILE_R",
                                     "GALVATRON_DP_FUSED", "GALVATRON_DP_SPLIT")):
        pytest.skip("the environment presets the layout")
    monkeypatch.setenv("GALVATRON_DP_TILE_TS", "11")
    monkeypatch.setenv("GALVATRON_DP_TILE_R", "1")
    monkeypatch.setenv("GALVATRON_DP_SPLIT", "2")
    rng = np.random.Generator(np.random.PCG64(4242))
    insts = [W.random_instance(rng, L, 44, V, mem_hi=max(1, V // (L + 1)), integer_costs=bool(n % 2), per_layer_inter=bool(n % 3),
                               inf_frac=0.1 * (n % 2), n_keys=3)
             for n, (L, V) in enumerate([(9, 3000), (4, 700), (9, 5000), (2, 129), (6, 2048), (1, 64)])]
    probs = []
    for inst in insts:
        keys = sorted(inst.other_mem)
        probs.append(_lib.Problem(inst.mem, inst.intra, inst.inter_tables, inst.V, [inst.other_mem[k] for k in keys],
                                  [inst.other_time[k] for k in keys], inter_index=inst.inter_index, launch="fused"))
    with _lib.Plan(probs) as plan:
        plan.set_option(_lib.GDP_OPT_POISON, 1)
        t = plan.run(1)
        assert t.fused == 1 and t.fused_split == 2
        plan.fetch()
    for n, (inst, prob) in enumerate(zip(insts, probs)):
        keys = sorted(inst.other_mem)
        want = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time)
        got = ({k: prob.total[i] for i, k in enumerate(keys)},
               {k: [int(x) for x in prob.res[i]] for i, k in enumerate(keys)},
               {k: int(prob.remaining[i]) for i, k in enumerate(keys)})
        H.assert_same_results(got, want, f"instance {n}")


@pytest.mark.parametrize("seed,shape", list(enumerate([(8, 17, 1), (12, 31, 65), (9, 8, 5), (6, 40, 64), (13, 5, 3), (10, 22, 7)])))
def test_keys_whose_reference_walk_leaves_the_table_are_reported_infeasible(seed, shape):
    """With memory costs of 0 and a budget of a few bins the reference's walk back can arrive at a negative
    row and index its argmin table with it (undefined behaviour, csrc/dp_core.cpp:105-113).  The library walks
    the same way but stops there: such a key comes back as infeasible (+inf, -1, strategy list untouched);
    every other key equals the reference's, costs-only and with the argmin table."""
    L, S, V = shape
    inst = W.zero_memory_tiny_budget(seed, L, S, V)
    undefined = set()
    want = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time, undefined=undefined)
    keys = sorted(inst.other_mem)
    for keep_marks in (False, True):
        prob = _lib.Problem(inst.mem, inst.intra, inst.inter_tables, inst.V, [inst.other_mem[k] for k in keys],
                            [inst.other_time[k] for k in keys], inter_index=inst.inter_index, keep_marks=keep_marks)
        _lib.solve_batch([prob])
        for i, k in enumerate(keys):
            if k in undefined:
                assert prob.total[i] == np.inf and prob.remaining[i] == -1 and (prob.res[i] == -1).all(), (k, prob.total[i])
            else:
                assert np.float64(prob.total[i]).tobytes() == np.float64(want[0][k]).tobytes(), (k, prob.total[i], want[0][k])
                assert int(prob.remaining[i]) == want[2][k]
                assert want[2][k] == -1 or [int(x) for x in prob.res[i]] == want[1][k]
