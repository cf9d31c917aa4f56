"""Shared helpers of the test-suite: golden case rebuilding and result comparison."""
import hashlib
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))

import make_golden  # noqa: E402  (tests/golden/make_golden.py: case builders only; it never needs the reference here)


def build_case(rec):
    inst = make_golden.build_case(rec["builder"], rec["kwargs"])
    assert inst.digest() == rec["input_sha256"], "generator no longer reproduces the fixture's inputs"
    return inst


def golden_results(rec):
    keys = rec["keys"]
    total = {k: float.fromhex(h) for k, h in zip(keys, rec["total_hex"])}
    rem = {k: r for k, r in zip(keys, rec["remaining"])}
    res = {k: list(r) for k, r in zip(keys, rec["res"])}
    return total, res, rem


def same_float(a, b):
    """Bit-exact equality of two doubles (inf == inf, 0.0 vs -0.0 differ)."""
    return np.float64(a).tobytes() == np.float64(b).tobytes()


def assert_same_results(got, want, ctx=""):
    gt, gr, gm = got
    wt, wr, wm = want
    assert list(gt) == list(wt), f"{ctx}: key order {list(gt)} != {list(wt)}"
    for k in wt:
        assert same_float(gt[k], wt[k]), f"{ctx}: total[{k}] {float(gt[k]).hex()} != {float(wt[k]).hex()}"
        assert int(gm[k]) == int(wm[k]), f"{ctx}: remaining[{k}] {gm[k]} != {wm[k]}"
        assert [int(x) for x in gr[k]] == [int(x) for x in wr[k]], f"{ctx}: res[{k}] differs"


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def hip_solve(inst, export=False):
    """Run one instance through the shim exactly as DPAlg.fit calls the plugin
    (dynamic_programming.py:78-92)."""
    import galvatron_dp_core as shim
    L, S, V = inst.L, inst.S, inst.V
    f = np.full((V, S), 0, dtype=np.float64) if inst.f0 is None else np.array(inst.f0, dtype=np.float64, order="C")
    mark = np.full((L, V, S), -1, dtype=np.int32) if export else np.zeros((1, 1, 1), dtype=np.int32)
    res = {k: np.full(L, -1, dtype=np.int32) for k in inst.other_mem}
    shim.set_export(export)
    try:
        total, rem = shim.dynamic_programming_core(L, V, S, inst.mem, mark, f, inst.inter, inst.intra,
                                                   inst.other_mem, inst.other_time, res)
    finally:
        shim.set_export(False)
    out = (total, {k: [int(x) for x in v] for k, v in res.items()}, rem)
    if export:
        return out + (f, mark)
    return out
