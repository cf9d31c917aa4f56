"""The C oracle against (a) the reference's own dp_core compiled into oracle/_ref, where that
build exists, and (b) the committed golden vectors written from it (tests/golden)."""
import numpy as np
import pytest

import helpers as H
from galvatron_dp import workloads as W
from oracle import dp_oracle as O

needs_ref = pytest.mark.skipif(not O.ref_available(), reason="oracle/_ref not built (no /root/reference)")

CPU_GOLDEN = ([f"ties_{i}" for i in range(10)] + [f"rand_{i}" for i in range(10)] +
              [f"infeasible_{i}" for i in range(10)] + [f"cfg3_smallV_{i}" for i in range(8)] +
              ["cfg2_small", "cfg4_small", "galvatron_like", "cfg0", "cfg0_other_time", "cfg1"] +
              [f"zeromem_{i}" for i in range(8)] + [f"initf_{i}" for i in range(8)] + ["initf_galvatron_like"])


@pytest.mark.parametrize("name", CPU_GOLDEN)
def test_oracle_matches_golden(golden, name):
    rec = golden[name]
    inst = H.build_case(rec)
    total, res, rem, f, mark = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time,
                                       f0=inst.f0, keep=True)
    H.assert_same_results((total, res, rem), H.golden_results(rec), name)
    assert H.sha(f) == rec["f_sha256"]
    assert H.sha(mark) == rec["mark_sha256"]


@pytest.mark.slow
@pytest.mark.parametrize("name", ["cfg2", "cfg4"] + [f"cfg3_{i:03d}" for i in (0, 100, 255)])
def test_oracle_matches_golden_full_size(golden, name):
    rec = golden[name]
    inst = H.build_case(rec)
    total, res, rem, f, mark = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time,
                                       keep=True)
    H.assert_same_results((total, res, rem), H.golden_results(rec), name)
    assert H.sha(f) == rec["f_sha256"] and H.sha(mark) == rec["mark_sha256"]


def test_golden_covers_every_benchmark_config(golden):
    for name in ["cfg0", "cfg1", "cfg2", "cfg4"] + [f"cfg3_{i:03d}" for i in range(256)]:
        assert name in golden, name


@needs_ref
@pytest.mark.parametrize("seed", range(20))
def test_oracle_vs_reference_build_random(seed):
    rng = np.random.Generator(np.random.PCG64(900 + seed))
    L, S, V = int(rng.integers(1, 9)), int(rng.integers(1, 70)), int(rng.integers(20, 900))
    inst = W.random_instance(rng, L, S, V, integer_costs=bool(seed % 2), mem_hi=max(1, V // (L + 1)),
                             mem_lo=0 if seed % 5 == 0 else 1,     # memory costs of 0: the in-place update reads its own row
                             inf_frac=0.15 * (seed % 3 == 0), over_frac=0.1 * (seed % 4 == 0), n_keys=4)
    a = O.solve(inst.mem, inst.intra, inst.inter, V, inst.other_mem, inst.other_time, keep=True)
    b = O.ref_solve(inst.mem, inst.intra, inst.inter, V, inst.other_mem, inst.other_time, keep=True)
    H.assert_same_results(a[:3], b[:3], f"seed {seed}")
    assert a[3].tobytes() == b[3].tobytes() and np.array_equal(a[4], b[4])


@needs_ref
@pytest.mark.parametrize("seed", range(12))
def test_oracle_vs_reference_build_with_initial_costs(seed):
    """``_f`` is read, not only written: the reference relaxes in place from whatever the caller's array
    holds (csrc/dp_core.cpp:46-47,67).  Random finite / +inf initial costs, memory costs of 0 included."""
    rng = np.random.Generator(np.random.PCG64(1700 + seed))
    L, S, V = int(rng.integers(1, 8)), int(rng.integers(1, 70)), int(rng.integers(20, 700))
    inst = W.random_instance(rng, L, S, V, integer_costs=bool(seed % 2), mem_hi=max(1, V // (L + 1)),
                             mem_lo=0 if seed % 4 == 0 else 1, inf_frac=0.1 * (seed % 3 == 0), n_keys=4)
    W.with_initial_costs(inst, rng, integer=bool(seed % 2), inf_frac=0.1 * (seed % 5 == 0))
    a = O.solve(inst.mem, inst.intra, inst.inter, V, inst.other_mem, inst.other_time, f0=inst.f0, keep=True)
    b = O.ref_solve(inst.mem, inst.intra, inst.inter, V, inst.other_mem, inst.other_time, f0=inst.f0, keep=True)
    H.assert_same_results(a[:3], b[:3], f"seed {seed}")
    assert a[3].tobytes() == b[3].tobytes() and np.array_equal(a[4], b[4])


@needs_ref
def test_int8_marks_equal_int32_marks():
    rng = np.random.Generator(np.random.PCG64(4))
    inst = W.random_instance(rng, 5, 30, 400, mem_hi=60)
    a = O.solve(inst.mem, inst.intra, inst.inter, 400, inst.other_mem, inst.other_time, keep=True)
    b = O.solve(inst.mem, inst.intra, inst.inter, 400, inst.other_mem, inst.other_time, keep=True, mark_dtype=np.int8)
    assert a[:3] == b[:3] and np.array_equal(a[4], b[4].astype(np.int32))
