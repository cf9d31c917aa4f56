"""Writes tests/golden/dp_core_golden.json from the reference's compiled dp_core.

Run in the build container only (it needs oracle/_ref, i.e. /root/reference):

    python oracle/build.py && python tests/golden/make_golden.py [--only NAME ...] [--jobs N]

For every case the seeded generator (galvatron_dp.workloads) rebuilds the inputs, the
reference's ``dynamic_programming_core`` (csrc/dp_core.cpp:24-120, compiled by
oracle/build.py) solves them exactly as ``DPAlg.fit`` calls it, and the fixture keeps
only data: the generator call, a SHA-256 of the input bytes, the per-key total cost
(hex float), strategy list and remaining memory, and SHA-256 digests of the final ``f``
[V,S] f64 and ``mark`` [L,V,S] int32 arrays in the reference's layouts.
"""
from __future__ import annotations

import argparse
import hashlib
import json
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "hetu-galvatron_amd"))

from galvatron_dp import workloads as W  # noqa: E402

OUT = os.path.join(HERE, "dp_core_golden.json")


def cases():
    """name -> (builder name, kwargs).  Builders are looked up in ``golden_cases``."""
    c = {}
    c["cfg0"] = ("config0", {})
    c["cfg0_other_time"] = ("config0", {"random_other_time": True})
    c["cfg1"] = ("config1", {})
    c["cfg2"] = ("config2", {})
    c["cfg2_small"] = ("config2", {"L": 12, "S": 64, "V": 12288})
    c["cfg4"] = ("config4", {})
    c["cfg4_small"] = ("config4", {"V": 16384, "n_each": 5})
    for i in range(256):
        c[f"cfg3_{i:03d}"] = ("config3_item", {"i": i})
    for i in range(8):
        c[f"cfg3_smallV_{i}"] = ("config3_item", {"i": 35 * i + 3, "V": 8192})
    # tie-heavy and edge cases (small enough for the CPU suite)
    for i, (L, S, V) in enumerate([(6, 5, 300), (9, 22, 700), (5, 64, 500), (4, 65, 400), (7, 3, 257),
                                   (3, 127, 300), (12, 44, 1500), (2, 1, 64), (1, 7, 100), (5, 88, 640)]):
        c[f"ties_{i}"] = ("ties", {"seed": 1000 + i, "L": L, "S": S, "V": V})
        c[f"rand_{i}"] = ("rand", {"seed": 2000 + i, "L": L, "S": S, "V": V})
        c[f"infeasible_{i}"] = ("infeasible", {"seed": 3000 + i, "L": L, "S": S, "V": V})
    c["galvatron_like"] = ("galvatron_like", {})
    # memory costs of 0: the in-place update then reads its own, partly updated row (csrc/dp_core.cpp:58-73)
    for i, (L, S, V, hi) in enumerate([(4, 6, 60, 2), (6, 22, 400, 3), (5, 44, 900, 1), (8, 64, 700, 4), (3, 65, 300, 2),
                                       (7, 9, 513, 0), (10, 40, 2000, 6), (2, 88, 640, 1)]):
        c[f"zeromem_{i}"] = ("zeromem", {"seed": 4000 + i, "L": L, "S": S, "V": V, "mem_hi": hi})
    # a non-zero ``_f`` on entry: the relaxation starts from it (csrc/dp_core.cpp:46-47,67)
    for i, (L, S, V, zero_mem) in enumerate([(3, 5, 200, False), (6, 22, 900, False), (5, 44, 1500, False), (4, 64, 2048, False),
                                             (7, 40, 3000, False), (3, 88, 700, False), (5, 22, 600, True), (4, 65, 500, True)]):
        c[f"initf_{i}"] = ("initial_f", {"seed": 5000 + i, "L": L, "S": S, "V": V, "zero_mem": zero_mem})
    c["initf_galvatron_like"] = ("initial_f_galvatron_like", {})
    return c


def build_case(builder: str, kw: dict) -> W.Instance:
    if builder == "config3_item":
        kw = dict(kw)
        i = kw.pop("i")
        return W.config3(n_limit=i + 1, **kw)[i]
    if builder == "ties":
        rng = np.random.Generator(np.random.PCG64(kw["seed"]))
        inst = W.random_instance(rng, kw["L"], kw["S"], kw["V"], integer_costs=True,
                                 mem_hi=max(1, kw["V"] // (kw["L"] + 1)), per_layer_inter=bool(kw["seed"] % 2))
        # duplicate a strategy so that exact ties between columns exist
        if kw["S"] >= 3:
            inst.mem[:, -1] = inst.mem[:, 0]
            inst.intra[:, -1] = inst.intra[:, 0]
            inter = np.array(inst.inter)
            inter[:, -1, :] = inter[:, 0, :]
            inter[:, :, -1] = inter[:, :, 0]
            inst.inter = inter
            inst.inter_tables, inst.inter_index = inter, np.arange(kw["L"], dtype=np.int32)
        return inst
    if builder == "rand":
        rng = np.random.Generator(np.random.PCG64(kw["seed"]))
        return W.random_instance(rng, kw["L"], kw["S"], kw["V"], mem_hi=max(1, kw["V"] // max(2, kw["L"] - 1)))
    if builder == "infeasible":
        rng = np.random.Generator(np.random.PCG64(kw["seed"]))
        return W.random_instance(rng, kw["L"], kw["S"], kw["V"], mem_hi=max(1, kw["V"] // (kw["L"] + 1)),
                                 inf_frac=0.2, over_frac=0.15, n_keys=4)
    if builder == "zeromem":
        rng = np.random.Generator(np.random.PCG64(kw["seed"]))
        # many zeros (mem in [0, mem_hi]), integer costs in the odd cases so that ties meet the in-row order
        inst = W.random_instance(rng, kw["L"], kw["S"], kw["V"], mem_lo=0, mem_hi=kw["mem_hi"],
                                 integer_costs=bool(kw["seed"] % 2), inf_frac=0.1 * (kw["seed"] % 3 == 0))
        if kw["seed"] % 4 == 1:                          # some strategies with ordinary costs among the zeros
            big = rng.uniform(size=inst.mem.shape) < 0.3
            inst.mem[big] = rng.integers(1, max(2, kw["V"] // (kw["L"] + 1)), size=int(big.sum()))
        return inst
    if builder == "initial_f":
        rng = np.random.Generator(np.random.PCG64(kw["seed"]))
        inst = W.random_instance(rng, kw["L"], kw["S"], kw["V"], mem_lo=0 if kw["zero_mem"] else 1,
                                 mem_hi=max(2, kw["V"] // (kw["L"] + 1)), integer_costs=bool(kw["seed"] % 2),
                                 per_layer_inter=bool(kw["seed"] % 3), inf_frac=0.1 * (kw["seed"] % 4 == 0), n_keys=4)
        return W.with_initial_costs(inst, rng, integer=bool(kw["seed"] % 2), inf_frac=0.05 * (kw["seed"] % 2 == 0))
    if builder == "initial_f_galvatron_like":
        return W.with_initial_costs(W.galvatron_like(), np.random.Generator(np.random.PCG64(78)), inf_frac=0.01)
    if builder == "galvatron_like":
        return W.galvatron_like()
    return getattr(W, builder)(**kw)


def solve_case(item):
    name, (builder, kw) = item
    from oracle import dp_oracle as O
    inst = build_case(builder, kw)
    t0 = time.time()
    total, res, rem, f, mark = O.ref_solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem,
                                           inst.other_time, f0=inst.f0, keep=True)
    dt = time.time() - t0
    keys = sorted(total)
    rec = {
        "builder": builder, "kwargs": kw, "L": inst.L, "S": inst.S, "V": inst.V,
        "input_sha256": inst.digest(), "keys": keys,
        "total_hex": [float(total[k]).hex() for k in keys],
        "remaining": [int(rem[k]) for k in keys],
        "res": [res[k] for k in keys],
        "f_sha256": hashlib.sha256(f.tobytes()).hexdigest(),
        "mark_sha256": hashlib.sha256(mark.tobytes()).hexdigest(),
        "ref_seconds": round(dt, 3),
    }
    print(f"{name}: {dt:.1f}s", flush=True)
    return name, rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--only", nargs="*", default=None, help="case-name prefixes to (re)generate")
    ap.add_argument("--jobs", type=int, default=1)
    a = ap.parse_args()
    todo = cases()
    if a.only:
        todo = {k: v for k, v in todo.items() if any(k.startswith(p) for p in a.only)}
    gold = {}
    if os.path.exists(OUT):
        with open(OUT) as fh:
            gold = json.load(fh)
    if a.jobs > 1:
        import multiprocessing as mp
        with mp.get_context("fork").Pool(a.jobs) as pool:
            for name, rec in pool.imap_unordered(solve_case, list(todo.items())):
                gold[name] = rec
    else:
        for item in todo.items():
            name, rec = solve_case(item)
            gold[name] = rec
    with open(OUT, "w") as fh:
        json.dump({k: gold[k] for k in sorted(gold)}, fh, indent=0, separators=(",", ":"))
    print("wrote", OUT, len(gold), "cases")


if __name__ == "__main__":
    main()
