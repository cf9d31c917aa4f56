"""GPU tests of the dense [L,S,S] transition array, as the reference's callers pass it
(galvatron/core/search_engine/dynamic_programming.py:368-372: one matrix per layer type repeated for
its layers, the first layer's zeroed): the library keeps matrices with equal bytes once.  Results must
be those of the oracle on the array as given, under every launch scheme."""
import os

import numpy as np
import pytest

import helpers as H
from galvatron_dp import _lib, workloads as W

pytestmark = pytest.mark.gpu

_PRESETS = ("GALVATRON_DP_KEEP_MARKS", "GALVATRON_DP_TILE_TS", "GALVATRON_DP_TILE_R", "GALVATRON_DP_FUSED",
            "GALVATRON_DP_LATENCY_VARIANT", "GALVATRON_DP_FLOW")

# which of a few random matrices each layer gets: all equal; the reference's shape (layer 0 of its own,
# then two layer types); runs, a matrix that comes back, and more different ones than are looked back at
_PATTERNS = {
    "all_equal": [0] * 12,
    "two_layer_types": [0] + [1] * 7 + [2] * 8,
    "mixed": [0, 0, 1, 1, 0, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 11, 3, 10, 0, 12, 12, 12, 1, 13],
    "all_different": list(range(10)),
}


def _results(prob, keys):
    return ({k: prob.total[i] for i, k in enumerate(keys)}, {k: [int(x) for x in prob.res[i]] for i, k in enumerate(keys)},
            {k: int(prob.remaining[i]) for i, k in enumerate(keys)})


@pytest.mark.parametrize("pattern", sorted(_PATTERNS))
@pytest.mark.parametrize("S,V", [(6, 700), (44, 3000)])
def test_dense_array_with_repeated_matrices(pattern, S, V, monkeypatch):
    if any(k in os.environ for k in _PRESETS):
        pytest.skip("the environment presets the layout")
    from oracle import dp_oracle as O
    which = _PATTERNS[pattern]
    L = len(which)
    rng = np.random.Generator(np.random.PCG64([23, S, L]))
    inst = W.random_instance(rng, L, S, V, mem_hi=V // 8, inf_frac=0.05, n_keys=2)
    mats = rng.uniform(0.0, 6.0, size=(max(which) + 1, S, S))
    if pattern == "two_layer_types":
        mats[0] = 0.0
    dense = np.ascontiguousarray(mats[which])
    if pattern == "mixed":
        dense[16, S - 1, S - 1] = np.nextafter(dense[16, S - 1, S - 1], 7.0)   # equal to matrix 3 but for its last entry
    wt, wr, wm, wf, wmark = O.solve(inst.mem, inst.intra, dense, inst.V, inst.other_mem, inst.other_time, keep=True)
    keys = sorted(inst.other_mem)
    om, ot = [inst.other_mem[k] for k in keys], [inst.other_time[k] for k in keys]
    for env in ({}, {"GALVATRON_DP_FUSED": "1"}, {"GALVATRON_DP_FUSED": "0", "GALVATRON_DP_FLOW": "0"},
                {"GALVATRON_DP_KEEP_MARKS": "1"}):
        for k in _PRESETS:
            monkeypatch.delenv(k, raising=False)
        for k, v in env.items():
            monkeypatch.setenv(k, v)
        for export in (False, True):
            prob = _lib.Problem(inst.mem, inst.intra, dense, inst.V, om, ot, export_f=export, export_mark=export)
            _lib.solve_batch([prob])
            H.assert_same_results(_results(prob, keys), (wt, wr, wm), f"{pattern} S={S} {env} export={export}")
            if export:
                assert prob.f_out.tobytes() == wf.tobytes()
                assert prob.mark_out.tobytes() == np.ascontiguousarray(wmark, dtype=np.int32).tobytes()


def test_dense_array_through_the_plugin_signature(golden):
    """cfg1 as the reference's caller would pass it (32 copies of one matrix): same results as the golden."""
    rec = golden["cfg1"]
    inst = H.build_case(rec)
    assert inst.inter.shape == (inst.L, inst.S, inst.S)
    H.assert_same_results(H.hip_solve(inst), H.golden_results(rec), "cfg1 dense")


def test_instances_of_a_batch_that_were_handed_the_same_matrices(monkeypatch):
    """Instances that point at the same transition matrices read one device copy: a batch that mixes
    instances sharing a table (with an index), instances sharing a dense array (one of them a shorter
    prefix of it), and instances with matrices of their own, under every launch scheme, against the
    oracle instance by instance."""
    if any(k in os.environ for k in _PRESETS):
        pytest.skip("the environment presets the layout")
    from oracle import dp_oracle as O
    rng = np.random.Generator(np.random.PCG64(31))
    S, V = 12, 900
    tables = np.ascontiguousarray(rng.uniform(0.0, 6.0, size=(3, S, S)))
    dense = np.ascontiguousarray(tables[[0, 0, 1, 1, 1, 2]])
    other = np.ascontiguousarray(rng.uniform(0.0, 6.0, size=(2, S, S)))
    specs = [("index", tables, [0, 1, 1, 2, 2]), ("index", tables, [2, 2, 0]), ("index", tables, [1, 0, 0, 0, 2, 2, 1]),
             ("dense", dense, None), ("dense", dense[:4], None), ("dense", dense[:6], None),
             ("index", other, [0, 1, 0, 1]), ("dense", np.ascontiguousarray(tables[[1, 1, 1]]), None)]
    probs, wants = [], []
    for kind, arr, index in specs:
        L = len(index) if index is not None else arr.shape[0]
        inst = W.random_instance(rng, L, S, V, mem_hi=V // 6, inf_frac=0.05, n_keys=2)
        full = arr[index] if index is not None else arr
        wants.append(O.solve(inst.mem, inst.intra, full, inst.V, inst.other_mem, inst.other_time))
        keys = sorted(inst.other_mem)
        om, ot = [inst.other_mem[k] for k in keys], [inst.other_time[k] for k in keys]
        probs.append((keys, lambda kind=kind, arr=arr, index=index, inst=inst, om=om, ot=ot: _lib.Problem(
            inst.mem, inst.intra, arr, inst.V, om, ot,
            inter_index=None if index is None else np.asarray(index, dtype=np.int32))))
    for env in ({}, {"GALVATRON_DP_FUSED": "1"}, {"GALVATRON_DP_FUSED": "0", "GALVATRON_DP_FLOW": "0"},
                {"GALVATRON_DP_KEEP_MARKS": "1"}):
        for k in _PRESETS:
            monkeypatch.delenv(k, raising=False)
        for k, v in env.items():
            monkeypatch.setenv(k, v)
        built = [make() for _, make in probs]
        _lib.check_layout(built)
        _lib.solve_batch(built)
        for n, ((keys, _), prob, want) in enumerate(zip(probs, built, wants)):
            H.assert_same_results(_results(prob, keys), want, f"instance {n} {env}")
