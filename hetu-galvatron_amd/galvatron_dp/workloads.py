"""Seeded synthetic DP instances for the five benchmark configurations.

Every instance is the argument set of one ``DPAlg.fit`` plugin call
(``galvatron/core/search_engine/dynamic_programming.py:79-91``): ``mem`` int32 [L,S]
(the reference's ``v_data``), ``intra`` f64 [L,S], ``inter`` f64 [L,S,S] (row = source
strategy, column = target strategy), number of budget bins ``V`` (the reference's
``max_mem`` argument) and the per-key ``other_mem`` / ``other_time`` dictionaries.

All draws come from ``numpy.random.Generator(PCG64(seed))`` in a fixed order, so an
instance is reproducible from ``(config, seed)`` alone; ``digest`` gives the SHA-256
of the arrays for checking that two machines built the same bytes.
"""
from __future__ import annotations

import hashlib
from dataclasses import dataclass, field

import numpy as np

DEFAULT_SEED = 20241125


@dataclass
class Instance:
    name: str
    mem: np.ndarray          # int32 [L,S]
    intra: np.ndarray        # f64   [L,S]
    inter: np.ndarray        # f64   [L,S,S]  (may be a broadcast view of [T,S,S][index])
    V: int                   # number of budget bins (reference argument ``max_mem``)
    other_mem: dict = field(default_factory=dict)
    other_time: dict = field(default_factory=dict)
    inter_tables: np.ndarray | None = None   # f64 [T,S,S] when layers share matrices
    inter_index: np.ndarray | None = None    # int32 [L] into inter_tables
    f0: np.ndarray | None = None             # f64 [V,S] contents of ``_f`` on entry (None: zeros, as DPAlg passes)

    @property
    def L(self) -> int:
        return int(self.mem.shape[0])

    @property
    def S(self) -> int:
        return int(self.mem.shape[1])

    @property
    def relaxations(self) -> int:
        return self.L * self.V * self.S * self.S

    def digest(self) -> str:
        h = hashlib.sha256()
        h.update(np.ascontiguousarray(self.mem, dtype=np.int32).tobytes())
        h.update(np.ascontiguousarray(self.intra, dtype=np.float64).tobytes())
        h.update(np.ascontiguousarray(self.inter, dtype=np.float64).tobytes())
        h.update(np.array([self.V], dtype=np.int64).tobytes())
        for k in sorted(self.other_mem):
            h.update(np.array([k, self.other_mem[k]], dtype=np.int64).tobytes())
            h.update(np.array([self.other_time[k]], dtype=np.float64).tobytes())
        if self.f0 is not None:
            h.update(np.ascontiguousarray(self.f0, dtype=np.float64).tobytes())
        return h.hexdigest()


def _keys(V: int, rng=None):
    other_mem = {1: 0, 2: V // 64, 4: V // 16, 8: V // 4}
    if rng is None:
        other_time = {k: 0.0 for k in other_mem}
    else:
        other_time = {k: float(rng.uniform(0.0, 50.0)) for k in other_mem}
    return other_mem, other_time


def _inter_matrix(rng, S: int, hi: float) -> np.ndarray:
    m = rng.uniform(0.0, hi, size=(S, S))
    np.fill_diagonal(m, 0.0)
    return m


def _shared(tables: np.ndarray, index: np.ndarray) -> np.ndarray:
    return tables[index]


def config0(seed: int = DEFAULT_SEED, random_other_time: bool = False) -> Instance:
    """L=24 identical layers, S=22, V=16384."""
    rng = np.random.Generator(np.random.PCG64(seed))
    L, S, V = 24, 22, 16384
    mem_row = rng.integers(100, 1201, size=S, dtype=np.int64).astype(np.int32)
    intra_row = rng.uniform(1.0, 20.0, size=S)
    tables = _inter_matrix(rng, S, 5.0)[None]
    index = np.zeros(L, dtype=np.int32)
    om, ot = _keys(V, rng if random_other_time else None)
    return Instance("cfg0", np.repeat(mem_row[None], L, 0), np.repeat(intra_row[None], L, 0),
                    _shared(tables, index), V, om, ot, tables, index)


def _layout_ckpt(rng, L: int, lo: int, hi: int, tlo: float, thi: float):
    base_mem = rng.integers(lo, hi + 1, size=(L, 22), dtype=np.int64)
    base_t = rng.uniform(tlo, thi, size=(L, 22))
    mem = np.concatenate([base_mem, np.ceil(0.4 * base_mem).astype(np.int64)], axis=1).astype(np.int32)
    intra = np.concatenate([base_t, 1.33 * base_t], axis=1)
    return mem, intra


def config1(seed: int = DEFAULT_SEED + 1, random_other_time: bool = False) -> Instance:
    """L=32, S=44 (22 layouts x checkpoint off/on), V=65536."""
    rng = np.random.Generator(np.random.PCG64(seed))
    L, S, V = 32, 44, 65536
    mem, intra = _layout_ckpt(rng, L, 200, 4000, 2.0, 40.0)
    tables = _inter_matrix(rng, S, 5.0)[None]
    index = np.zeros(L, dtype=np.int32)
    om, ot = _keys(V, rng if random_other_time else None)
    return Instance("cfg1", mem, intra, _shared(tables, index), V, om, ot, tables, index)


def config2(seed: int = DEFAULT_SEED + 2, random_other_time: bool = False,
            L: int = 80, S: int = 64, V: int = 131072) -> Instance:
    """L=80 heterogeneous layers, S=64, V=131072, one dense inter matrix per layer."""
    rng = np.random.Generator(np.random.PCG64(seed))
    mem = rng.integers(500, 8001, size=(L, S), dtype=np.int64).astype(np.int32)
    intra = rng.lognormal(2.5, 0.5, size=(L, S))
    tables = np.stack([_inter_matrix(rng, S, 10.0) for _ in range(L)])
    index = np.arange(L, dtype=np.int32)
    om, ot = _keys(V, rng if random_other_time else None)
    return Instance("cfg2", mem, intra, tables, V, om, ot, tables, index)


SWEEP_PP = (1, 2, 4, 8)
SWEEP_BSZ = tuple(range(8, 8 * 17, 8))      # 16 global batch sizes: 8..128
SWEEP_CHUNKS = (1, 2, 4, 8)


def config3(seed: int = DEFAULT_SEED + 3, n_limit: int | None = None, V: int = 65536) -> list[Instance]:
    """256 instances: pp x bsz x chunks, L=32/pp, S=44, one shared inter matrix."""
    rng0 = np.random.Generator(np.random.PCG64(seed))
    S = 44
    tables = _inter_matrix(rng0, S, 5.0)[None]
    out = []
    n = 0
    for pp in SWEEP_PP:
        for bsz in SWEEP_BSZ:
            for chunks in SWEEP_CHUNKS:
                if n_limit is not None and n >= n_limit:
                    return out
                rng = np.random.Generator(np.random.PCG64([seed, pp, bsz, chunks]))
                L = 32 // pp
                mem, intra = _layout_ckpt(rng, L, 200, 4000, 2.0, 40.0)
                intra = intra * (bsz / chunks)
                index = np.zeros(L, dtype=np.int32)
                om, ot = _keys(V)
                out.append(Instance(f"cfg3[pp{pp},bsz{bsz},ch{chunks}]", mem, intra, _shared(tables, index),
                                    V, om, ot, tables, index))
                n += 1
    return out


def config4(seed: int = DEFAULT_SEED + 4, random_other_time: bool = False,
            V: int = 262144, n_each: int = 24) -> Instance:
    """Encoder-decoder: 24+24 layers from two cost tables, S=88, about 15 % of the
    (layer, strategy) cells infeasible (mem above the budget, or intra = +inf)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    S, L = 88, 2 * n_each
    rows_mem = rng.integers(500, 8001, size=(2, S), dtype=np.int64)
    rows_t = rng.lognormal(2.5, 0.5, size=(2, S))
    tables = np.stack([_inter_matrix(rng, S, 10.0) for _ in range(2)])
    index = np.repeat(np.arange(2, dtype=np.int32), n_each)
    mem = rows_mem[index].copy()
    intra = rows_t[index].copy()
    bad = rng.uniform(size=(L, S)) < 0.15
    kind = rng.uniform(size=(L, S)) < 0.5
    over = V + rng.integers(1, 4097, size=(L, S), dtype=np.int64)
    mem = np.where(bad & kind, over, mem).astype(np.int32)
    intra = np.where(bad & ~kind, np.inf, intra)
    om, ot = _keys(V, rng if random_other_time else None)
    return Instance("cfg4", mem, intra, _shared(tables, index), V, om, ot, tables, index)


def galvatron_like() -> Instance:
    """Shape of a real search-engine call: 28 identical layers, inter made of zeros and
    the 1e-10..3e-9 ordering sentinels, first layer's inter zeroed, four keys
    (dynamic_programming.py:241,266,347-372).  Numbers are synthetic."""
    rng = np.random.Generator(np.random.PCG64(77))
    L, S, V = 28, 40, 29493
    mem_row = rng.integers(300, 2600, size=S)
    t_row = np.round(rng.uniform(20, 60, size=S), 3)
    m = np.zeros((S, S))
    sent = np.array([0.0, 1e-10, 1e-9, 2e-9, 3e-9, 0.37, 1.21])
    m[:] = sent[rng.integers(0, len(sent), size=(S, S))]
    np.fill_diagonal(m, 0.0)
    inter = np.repeat(m[None], L, 0)
    inter[0] = 0.0
    om = {1: 4100, 2: 2300, 4: 1500, 8: 900}
    ot = {1: 31.5, 2: 17.25, 4: 9.125, 8: 6.0625}
    return Instance("galvatron_like", np.repeat(mem_row[None], L, 0).astype(np.int32),
                      np.repeat(t_row[None], L, 0), inter, V, om, ot, inter, np.arange(L, dtype=np.int32))


CONFIGS = {0: config0, 1: config1, 2: config2, 3: config3, 4: config4}


def zero_memory_tiny_budget(seed: int, L: int, S: int, V: int) -> Instance:
    """Memory costs of 0 and 1 under a budget of a few bins: the in-place update then chains cells of one
    layer (csrc/dp_core.cpp:58-73), and the reference's walk back, which does not know that, can arrive at
    a negative row (csrc/dp_core.cpp:105-113)."""
    rng = np.random.Generator(np.random.PCG64([8, seed, L, S, V]))
    inst = random_instance(rng, L, S, V, mem_lo=0, mem_hi=max(1, V // (L + 1)), n_keys=4)
    inst.other_mem = {k: int(rng.integers(0, V)) for k in inst.other_mem}
    inst.other_mem[min(inst.other_mem)] = 0
    return inst


def with_initial_costs(inst: Instance, rng, *, integer: bool = False, inf_frac: float = 0.0) -> Instance:
    """``inst`` with a non-zero ``_f`` on entry: the reference relaxes in place from whatever the caller's
    array holds (csrc/dp_core.cpp:46-47,67).  Finite entries (small integers with ``integer``, so that
    they tie with the costs), a share ``inf_frac`` of +inf."""
    V, S = inst.V, inst.S
    f0 = rng.integers(0, 5, size=(V, S)).astype(np.float64) if integer else rng.uniform(-3.0, 25.0, size=(V, S))
    if inf_frac > 0:
        f0 = np.where(rng.uniform(size=(V, S)) < inf_frac, np.inf, f0)
    inst.f0 = np.ascontiguousarray(f0)
    return inst


def random_instance(rng, L: int, S: int, V: int, *, mem_lo=1, mem_hi=None, integer_costs=False,
                    per_layer_inter=True, inf_frac=0.0, over_frac=0.0, n_keys=3) -> Instance:
    """Small random instance for differential tests.  ``integer_costs`` makes costs small
    integers so that many paths tie exactly and the lowest-index rule decides."""
    mem_hi = max(mem_lo, V // 2) if mem_hi is None else mem_hi
    mem = rng.integers(mem_lo, mem_hi + 1, size=(L, S), dtype=np.int64)
    if integer_costs:
        intra = rng.integers(0, 4, size=(L, S)).astype(np.float64)
        T = L if per_layer_inter else 1
        tables = rng.integers(0, 3, size=(T, S, S)).astype(np.float64)
    else:
        intra = rng.uniform(0.5, 30.0, size=(L, S))
        T = L if per_layer_inter else 1
        tables = rng.uniform(0.0, 6.0, size=(T, S, S))
    index = np.arange(L, dtype=np.int32) if per_layer_inter else np.zeros(L, dtype=np.int32)
    if inf_frac > 0:
        intra = np.where(rng.uniform(size=(L, S)) < inf_frac, np.inf, intra)
    if over_frac > 0:
        mem = np.where(rng.uniform(size=(L, S)) < over_frac, V + rng.integers(0, 5, size=(L, S)), mem)
    keys = sorted(rng.choice(np.arange(1, 17), size=n_keys, replace=False).tolist())
    om = {int(k): int(rng.integers(0, V + 3)) for k in keys}
    om[int(keys[0])] = 0
    ot = {int(k): float(rng.uniform(0, 9)) for k in keys}
    return Instance("random", mem.astype(np.int32), intra, tables[index], V, om, ot, tables, index)
