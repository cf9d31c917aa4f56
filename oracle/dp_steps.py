"""Step form of the layer-wise DP on the CPU (TEST INFRASTRUCTURE ONLY, like everything under oracle/).

A second, independent restatement of ``csrc/dp_core.cpp:57-117``: instead of one cell per budget bin it
keeps every cost column ``f[.][s]`` as the list of its steps -- ``(first bin, cost, argmin)`` runs of equal
cells -- and evaluates the recurrence once per step.

Why that is the same computation, bit for bit.  The reference computes cell ``(v, s)`` of layer ``l`` from
row ``u = v - mem[l][s]`` of the previous layer alone (``csrc/dp_core.cpp:65-73``):
``cand[si] = (f[u][si] + inter[l][si][s]) + intra[l][s]``, first minimum under strict ``<``.  Two bins whose
source rows hold the same ``S`` values get the same candidates, hence the same cost and the same argmin.  The
source rows change only where some column has a step, so it is enough to evaluate one row per element of the
union of the columns' step positions; every other cell is a copy of the one below it.  The additions are the
same two IEEE-754 additions in the same order (numpy adds doubles elementwise), ``numpy.argmin`` returns the
first of equal minima and 0 for a row of ``+inf``, like ``std::min_element`` (``csrc/dp_core.cpp:12-16,70``).
Cells with ``v < mem[l][s]`` are ``+inf`` with argmin ``-1`` (``:60-64``).  Memory costs of 0 (the in-place
update then reads its own row) are not covered: this form is for ``mem >= 1``.

Used by tests/test_oracle_step_form.py against the dense restatement and the vectors written from the
reference's compiled dp_core, and to count how many relaxations a step-wise evaluation would carry out.
"""
from __future__ import annotations

import numpy as np


class Column:
    """``f[.][s]`` (and ``mark[l][.][s]``) as runs: run k covers bins ``start[k] .. start[k+1]-1``."""
    __slots__ = ("start", "cost", "arg")

    def __init__(self, start, cost, arg):
        self.start, self.cost, self.arg = start, cost, arg

    def at(self, v):
        k = np.searchsorted(self.start, v, side="right") - 1
        return self.cost[k], self.arg[k]


def _merge(start, cost, arg):
    """Drops a run that repeats its predecessor's cost and argmin."""
    if len(start) <= 1:
        return start, cost, arg
    keep = np.ones(len(start), dtype=bool)
    same_cost = (cost[1:] == cost[:-1]) | (np.isinf(cost[1:]) & np.isinf(cost[:-1]))
    keep[1:] = ~(same_cost & (arg[1:] == arg[:-1]))
    return start[keep], cost[keep], arg[keep]


def relax(mem, intra, inter, V, f0=None):
    """All layers.  Returns ``(columns per layer, stats per layer)``; ``columns[l][s]`` describes ``f`` after
    layer ``l`` for strategy ``s`` together with ``mark[l][.][s]``.  ``stats[l]`` = rows evaluated (the union of
    the source columns' steps), relaxations carried out, and the steps of the layer's output."""
    mem = np.asarray(mem, dtype=np.int64)
    intra = np.asarray(intra, dtype=np.float64)
    inter = np.asarray(inter, dtype=np.float64)
    L, S = mem.shape
    assert (mem >= 1).all(), "the step form does not cover memory costs of 0"
    if f0 is None:
        cols = [Column(np.zeros(1, np.int64), np.zeros(1), np.zeros(1, np.int64)) for _ in range(S)]
    else:
        f0 = np.asarray(f0, dtype=np.float64)
        cols = []
        for s in range(S):
            change = np.flatnonzero(np.r_[True, f0[1:, s] != f0[:-1, s]])
            cols.append(Column(change.astype(np.int64), f0[change, s].copy(), np.zeros(len(change), np.int64)))
    layers, stats = [], []
    for l in range(L):
        rows = np.unique(np.concatenate([c.start for c in cols]))           # source rows that differ from the row below
        src = np.empty((len(rows), S))
        for sp, c in enumerate(cols):
            src[:, sp] = c.cost[np.searchsorted(c.start, rows, side="right") - 1]
        new = []
        steps = 0
        for s in range(S):
            m = int(mem[l, s])
            cand = (src + inter[l][:, s][None, :]) + intra[l, s]             # (f + inter) + intra, csrc/dp_core.cpp:67
            arg = np.argmin(cand, axis=1)                                    # first minimum; 0 for a row of +inf
            cost = cand[np.arange(len(rows)), arg]
            start = rows + m                                                 # the cell that reads source row u is v = u + mem
            inside = start < V
            start, cost, arg = start[inside], cost[inside], arg[inside]
            head = min(m, V)                                                 # v < mem: +inf, argmin -1 (:60-64)
            start = np.r_[0, start]
            cost = np.r_[np.inf, cost]
            arg = np.r_[-1, arg]
            if head == 0:
                start, cost, arg = start[1:], cost[1:], arg[1:]
            start, cost, arg = _merge(start.astype(np.int64), cost, arg.astype(np.int64))
            new.append(Column(start, cost, arg))
            steps += len(start)
        cols = new
        layers.append(cols)
        stats.append({"rows": int(len(rows)), "relaxations": int(len(rows)) * S * S, "steps": steps})
    return layers, stats


def solve(mem, intra, inter, V, other_mem, other_time, f0=None):
    """``(total, res, remaining)`` dicts like ``dp_oracle.solve``, plus the per-layer statistics
    (epilogue: csrc/dp_core.cpp:78-117)."""
    mem = np.asarray(mem, dtype=np.int64)
    L, S = mem.shape
    layers, stats = relax(mem, intra, inter, V, f0)
    total, res, rem = {}, {}, {}
    for k in sorted(other_mem):
        total[k], res[k], rem[k] = float("inf"), [-1] * L, -1
        v = V - 1 - int(other_mem[k])
        if v < 0:
            continue
        last = np.array([layers[L - 1][s].at(v)[0] for s in range(S)])
        idx = int(np.argmin(last))
        if not last[idx] < np.inf:
            continue
        total[k] = float(last[idx] + other_time[k])
        path = [0] * L
        path[L - 1] = idx
        for i in range(L - 1, 0, -1):
            cur = idx
            idx = int(layers[i][cur].at(v)[1])
            v -= int(mem[i, cur])
            path[i - 1] = idx
        res[k] = path
        rem[k] = v - int(mem[0, idx])
    return total, res, rem, stats


def dense(layers, V):
    """``f`` [V,S] f64 after the last layer and ``mark`` [L,V,S] int32, expanded from the runs (for comparison
    with the reference's arrays)."""
    L, S = len(layers), len(layers[0])
    f = np.empty((V, S))
    mark = np.empty((L, V, S), dtype=np.int32)
    bins = np.arange(V)
    for l in range(L):
        for s, c in enumerate(layers[l]):
            k = np.searchsorted(c.start, bins, side="right") - 1
            mark[l, :, s] = c.arg[k]
            if l == L - 1:
                f[:, s] = c.cost[k]
    return f, mark
