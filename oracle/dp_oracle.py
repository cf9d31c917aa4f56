"""ctypes front end of the CPU checkers (TEST INFRASTRUCTURE ONLY).

``solve`` drives ``oracle/libdp_oracle.so`` (the plain-C restatement of
``csrc/dp_core.cpp:24-120``); ``ref_solve`` drives the reference's own translation
unit compiled into ``oracle/_ref`` with the argument list ``DPAlg.fit`` uses
(``galvatron/core/search_engine/dynamic_programming.py:76-94``).

Only tests, the smoke check and the bench's ``cpu_baseline`` leg may import this
module; the shipped library never does.
"""
from __future__ import annotations

import ctypes
import importlib.machinery
import importlib.util
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None
_ref = None

_i32p = ctypes.POINTER(ctypes.c_int32)
_i8p = ctypes.POINTER(ctypes.c_int8)
_i64p = ctypes.POINTER(ctypes.c_int64)
_f64p = ctypes.POINTER(ctypes.c_double)


def _ptr(a, typ):
    return None if a is None else a.ctypes.data_as(typ)


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(HERE, "libdp_oracle.so")
        if not os.path.exists(path):
            from oracle import build as _b
            _b.build_oracle()
        L = ctypes.CDLL(path)
        L.dp_oracle_solve.restype = None
        L.dp_oracle_solve.argtypes = [ctypes.c_int] * 3 + [_i32p, _f64p, _f64p, _f64p, _i32p, _i8p,
                                                         ctypes.c_int, _i64p, _f64p, _f64p, _i32p, _i32p]
        L.dp_oracle_walk_leaves_table.restype = ctypes.c_int
        L.dp_oracle_walk_leaves_table.argtypes = [ctypes.c_int] * 3 + [_i32p, _f64p, _i32p, _i8p, ctypes.c_int64]
        L.dp_oracle_relax.restype = None
        L.dp_oracle_relax.argtypes = [ctypes.c_int] * 3 + [_i32p, _f64p, _f64p, _f64p, _i32p, _i8p]
        L.dp_oracle_coarse.restype = None
        L.dp_oracle_coarse.argtypes = [ctypes.c_int] * 3 + [_i32p, _f64p, _f64p, _i32p, ctypes.c_int,
                                                           ctypes.c_int64, ctypes.c_double, _f64p, _i32p, _i32p]
        _lib = L
    return _lib


def solve(mem, intra, inter, V, other_mem, other_time, *, f0=None, mark_dtype=np.int32, keep=False, undefined=None):
    """Run the C restatement.  Returns ``(total, res, remaining)`` dicts keyed like
    ``other_mem`` (ascending), plus ``(f, mark)`` in the reference's layouts when
    ``keep`` is true.  ``mark_dtype`` int32 (reference) or int8 (compact).
    ``undefined``: a set that receives the keys for which the reference's walk back indexes its argmin table
    with a negative row -- possible only with memory costs of 0, undefined behaviour in the reference
    (csrc/dp_core.cpp:105-113), so their strategy list and remaining memory mean nothing."""
    mem = np.ascontiguousarray(mem, dtype=np.int32)
    intra = np.ascontiguousarray(intra, dtype=np.float64)
    inter = np.ascontiguousarray(inter, dtype=np.float64)
    L, S = mem.shape
    assert intra.shape == (L, S) and inter.shape == (L, S, S)
    f = np.zeros((V, S), dtype=np.float64) if f0 is None else np.array(f0, dtype=np.float64, order="C")
    mark = np.full((L, V, S), -1, dtype=mark_dtype)
    keys = sorted(other_mem)
    om = np.array([int(other_mem[k]) for k in keys], dtype=np.int64)
    ot = np.array([float(other_time[k]) for k in keys], dtype=np.float64)
    total = np.zeros(len(keys), dtype=np.float64)
    rem = np.zeros(len(keys), dtype=np.int32)
    res = np.full((len(keys), L), -1, dtype=np.int32)
    m32 = mark if mark_dtype == np.int32 else None
    m8 = mark if mark_dtype == np.int8 else None
    lib().dp_oracle_solve(L, V, S, _ptr(mem, _i32p), _ptr(intra, _f64p), _ptr(inter, _f64p), _ptr(f, _f64p),
                          _ptr(m32, _i32p), _ptr(m8, _i8p), len(keys), _ptr(om, _i64p), _ptr(ot, _f64p),
                          _ptr(total, _f64p), _ptr(rem, _i32p), _ptr(res, _i32p))
    if undefined is not None:
        for i, k in enumerate(keys):
            if lib().dp_oracle_walk_leaves_table(L, V, S, _ptr(mem, _i32p), _ptr(f, _f64p), _ptr(m32, _i32p), _ptr(m8, _i8p),
                                                 int(om[i])):
                undefined.add(k)
    out = ({k: float(total[i]) for i, k in enumerate(keys)},
           {k: [int(x) for x in res[i]] for i, k in enumerate(keys)},
           {k: int(rem[i]) for i, k in enumerate(keys)})
    if keep:
        return out + (f, mark)
    return out


def coarse(mem, intra, inter, V, strategy_tp, other_mem, other_time):
    """C restatement of the coarse branch (dynamic_programming.py:62-75)."""
    mem = np.ascontiguousarray(mem, dtype=np.int32)
    intra = np.ascontiguousarray(intra, dtype=np.float64)
    inter = np.ascontiguousarray(inter, dtype=np.float64)
    tp = np.ascontiguousarray(strategy_tp, dtype=np.int32)
    L, S = mem.shape
    total, res, rem = {}, {}, {}
    for k in other_mem:
        t = ctypes.c_double()
        r = ctypes.c_int32()
        path = np.full(L, -1, dtype=np.int32)
        lib().dp_oracle_coarse(L, V, S, _ptr(mem, _i32p), _ptr(intra, _f64p), _ptr(inter, _f64p), _ptr(tp, _i32p),
                               int(k), int(other_mem[k]), float(other_time[k]), ctypes.byref(t), ctypes.byref(r),
                               _ptr(path, _i32p))
        total[k], rem[k], res[k] = t.value, r.value, path
    return total, res, rem


def ref_available() -> bool:
    import sysconfig
    return os.path.exists(os.path.join(HERE, "_ref", "galvatron_dp_core" + sysconfig.get_config_var("EXT_SUFFIX")))


def ref_module():
    """The reference's pybind11 module built by oracle/build.py (not put in sys.modules,
    so it cannot shadow the shipped shim of the same name)."""
    global _ref
    if _ref is None:
        import sysconfig
        path = os.path.join(HERE, "_ref", "galvatron_dp_core" + sysconfig.get_config_var("EXT_SUFFIX"))
        loader = importlib.machinery.ExtensionFileLoader("galvatron_dp_core", path)
        spec = importlib.util.spec_from_file_location("galvatron_dp_core", path, loader=loader)
        mod = importlib.util.module_from_spec(spec)
        loader.exec_module(mod)
        _ref = mod
    return _ref


def ref_solve(mem, intra, inter, V, other_mem, other_time, *, f0=None, keep=False):
    """Call the reference's compiled ``dynamic_programming_core`` exactly as
    ``DPAlg.fit`` does (dynamic_programming.py:78-92).  ``f0``: what ``_f`` holds on entry
    (the reference relaxes in place from it, csrc/dp_core.cpp:46-47,67); None for DPAlg's zeros."""
    mem = np.ascontiguousarray(mem, dtype=np.int32)
    intra = np.ascontiguousarray(intra, dtype=np.float64)
    inter = np.ascontiguousarray(inter, dtype=np.float64)
    L, S = mem.shape
    f = np.full((V, S), 0, dtype=np.float64) if f0 is None else np.array(f0, dtype=np.float64, order="C")
    assert f.shape == (V, S)
    mark = np.full((L, V, S), -1, dtype=np.int32)
    res = {k: np.full(L, -1, dtype=np.int32) for k in other_mem}
    total, rem = ref_module().dynamic_programming_core(L, V, S, mem, mark, f, inter, intra,
                                                       {int(k): int(v) for k, v in other_mem.items()},
                                                       {int(k): float(v) for k, v in other_time.items()}, res)
    out = (dict(total), {k: [int(x) for x in v] for k, v in res.items()}, dict(rem))
    if keep:
        return out + (f, mark)
    return out
