"""Drop-in for the reference's compiled plugin module ``galvatron_dp_core``
(``PYBIND11_MODULE(galvatron_dp_core, ...)``, csrc/dp_core.cpp:122-124).

``DPAlg.fit`` does ``import galvatron_dp_core`` and calls
``galvatron_dp_core.dynamic_programming_core(...)`` with eleven positional arguments
(galvatron/core/search_engine/dynamic_programming.py:77-91).  Putting this file's directory on
``sys.path`` ahead of the reference's ``build/lib`` makes that call run on the MI355X through
libgalvatron_dp_hip.so; nothing else in the caller changes.

``_f`` is read as the reference reads it: the relaxation starts from whatever the array holds on entry
(csrc/dp_core.cpp:46-47,67; ``DPAlg`` hands in zeros, dynamic_programming.py:16), ``None`` standing for
zeros.

Differences from the compiled reference module, all on arguments no caller reads back:
``_mark`` and ``_f`` are filled only after ``set_export(True)`` (the argmin table lives on the
device in a compact form, and copying L*V*S int32 back per call would dominate the run time).
Inputs on which the reference's result depends on evaluation order or is undefined raise
``ValueError`` instead of computing something: NaN / -inf costs (also in ``_f``), a -0.0 in ``_f``,
negative memory costs, a negative ``other_mem_cost`` (start row above the table).  A memory cost of 0 is computed with the reference's
in-place order (csrc/dp_core.cpp:58-73); where the reference's walk back would then index its argmin table
with a negative row (undefined behaviour, csrc/dp_core.cpp:105-113) the key comes back as infeasible.
"""
from __future__ import annotations

import threading

import numpy as np

from galvatron_dp import _lib

__all__ = ["dynamic_programming_core", "dynamic_programming_core_batch", "set_export", "export_enabled", "SharedInter"]

_state = threading.local()      # per thread: the reference's parallel search calls the plugin from many threads


def set_export(flag: bool) -> None:
    """When true, the calls of THIS thread write ``_f`` and ``_mark`` exactly as the reference writes them
    (csrc/dp_core.cpp:61-62,72-73).  Other threads are not affected; ``dynamic_programming_core_batch`` also
    takes the choice per call (``export=``)."""
    _state.export = bool(flag)


def export_enabled() -> bool:
    """What ``set_export`` last set in the calling thread (False if it never did)."""
    return getattr(_state, "export", False)


class SharedInter:
    """``inter_cost`` of a call whose layers share a few transition matrices: ``tables`` f64 [T,S,S]
    and ``index`` int32 [L] (layer -> matrix), accepted wherever the plugin takes the reference's dense
    [L,S,S] array (no counterpart in the reference, which always passes the dense array).  The device
    then holds every matrix once."""
    __slots__ = ("tables", "index")

    def __init__(self, tables, index):
        self.tables = np.ascontiguousarray(tables, dtype=np.float64)
        self.index = np.ascontiguousarray(index, dtype=np.int32)

    def dense(self):
        return self.tables[self.index]

    def __getitem__(self, item):               # so that code written for the dense array can still slice it
        return self.dense()[item]


def _problem(layer_num, max_mem, strategy_num, v_data, _f, inter_cost, intra_cost, other_mem_cost, other_time_cost,
             export):
    L, V, S = int(layer_num), int(max_mem), int(strategy_num)
    mem = np.ascontiguousarray(v_data, dtype=np.int32).reshape(L, S)
    intra = np.ascontiguousarray(intra_cost, dtype=np.float64).reshape(L, S)
    keys = sorted(int(k) for k in other_mem_cost)          # std::map iterates in ascending key order
    om = [int(other_mem_cost[k]) for k in keys]
    ot = [float(other_time_cost[k]) if k in other_time_cost else 0.0 for k in keys]  # map::operator[] default
    if isinstance(inter_cost, SharedInter):
        return keys, _lib.Problem(mem, intra, inter_cost.tables.reshape(-1, S, S), V, om, ot,
                                  inter_index=inter_cost.index.reshape(L), export_f=export, export_mark=export,
                                  f0=_f)
    inter = np.ascontiguousarray(inter_cost, dtype=np.float64).reshape(L, S, S)
    return keys, _lib.Problem(mem, intra, inter, V, om, ot, export_f=export, export_mark=export, f0=_f)


def _finish(keys, prob, _mark, _f, res_list, export):
    total_cost, remaining_mem = {}, {}
    for i, k in enumerate(keys):
        total_cost[k] = float(prob.total[i])
        remaining_mem[k] = int(prob.remaining[i])
        if prob.remaining[i] != -1:
            res_list[k][...] = prob.res[i]                    # feasible keys only (csrc/dp_core.cpp:103-113)
    if export:
        np.asarray(_f)[...] = prob.f_out
        np.asarray(_mark)[...] = prob.mark_out
    return total_cost, remaining_mem


def dynamic_programming_core(layer_num, max_mem, strategy_num, v_data, _mark, _f, inter_cost, intra_cost,
                             other_mem_cost, other_time_cost, res_list):
    """Same signature and return value as the reference (csrc/dp_core.cpp:24-35,119):
    ``(total_cost: dict key->float, remaining_mem: dict key->int)``; ``res_list[key]`` (int32 [L],
    pre-filled with -1 by the caller) is written in place for feasible keys."""
    export = export_enabled()
    keys, prob = _problem(layer_num, max_mem, strategy_num, v_data, _f, inter_cost, intra_cost, other_mem_cost,
                          other_time_cost, export)
    _lib.solve_batch([prob])
    return _finish(keys, prob, _mark, _f, res_list, export)


def dynamic_programming_core_batch(calls, export=None):
    """Many reference calls in one device batch.  ``calls`` is a sequence of 11-tuples with the
    positional arguments of ``dynamic_programming_core``; returns the list of its return values.
    ``export``: write ``_f`` / ``_mark`` of every call (None: what ``set_export`` set in this thread)."""
    export = export_enabled() if export is None else bool(export)
    built = [_problem(c[0], c[1], c[2], c[3], c[5], c[6], c[7], c[8], c[9], export) for c in calls]
    _lib.solve_batch([b[1] for b in built])
    return [_finish(keys, prob, c[4], c[5], c[10], export) for (keys, prob), c in zip(built, calls)]
