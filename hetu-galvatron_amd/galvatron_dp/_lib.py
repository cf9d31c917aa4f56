"""ctypes binding of libgalvatron_dp_hip.so (the C ABI in include/galvatron_dp_hip.h).

There is no CPU fallback: if the HIP library has not been built, or no HIP device is usable,
every compute call raises.
"""
from __future__ import annotations

import ctypes
import os
from typing import Sequence

import numpy as np

PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# GALVATRON_DP_HIP_LIB points at another build of the same library (e.g. a tuning variant).
LIB_PATH = os.environ.get("GALVATRON_DP_HIP_LIB") or os.path.join(PKG, "lib", "libgalvatron_dp_hip.so")

GDP_OK = 0
GDP_E_BADARG = -1
GDP_E_UNSUPPORTED = -2
GDP_E_NONFINITE = -3
GDP_E_NOMEM = -4
GDP_E_HIP = -5
GDP_EXPORT_F = 1
GDP_EXPORT_MARK = 2
GDP_LAUNCH_FUSED = 4
GDP_LAUNCH_PER_LAYER = 8
GDP_COMPUTE_ALL = 16
GDP_KEEP_MARKS = 32
GDP_MAX_S = 1024
GDP_MAX_S_MARKS = 256
GDP_OPT_FUSED = 1
GDP_OPT_SPIN_LIMIT = 2
GDP_OPT_POISON = 3
GDP_OPT_NO_FALLBACK = 4
GDP_OPT_FLOW = 5
GDP_OPT_DEBUG_STALL = 6

GDP_STATIC_SCRATCH_BYTES = 64 << 20

EXPORTED_SYMBOLS = ("gdp_solve", "gdp_solve_batch", "gdp_solve_static", "gdp_plan_create", "gdp_plan_run", "gdp_plan_fetch",
                    "gdp_plan_destroy", "gdp_plan_set_option", "gdp_cache_trim", "gdp_last_error", "gdp_version",
                    "gdp_device_info", "gdp_debug_check_layout", "gdp_debug_shared_device", "gdp_batch_stats_begin",
                    "gdp_batch_stats_end")

_i32p = ctypes.POINTER(ctypes.c_int32)
_i64p = ctypes.POINTER(ctypes.c_int64)
_f64p = ctypes.POINTER(ctypes.c_double)


class UnsupportedInputError(ValueError):
    """GDP_E_UNSUPPORTED.  No input is answered with it any more (a memory cost of 0, once refused, is
    computed with the reference's in-place order); kept so that callers catching it keep working."""


# The pointer members are declared as untyped pointers (same layout as the typed ones of the header):
# they are then filled with plain addresses, which costs a fraction of a typed cast per array -- a sweep
# builds thousands of these records.
_ptr = ctypes.c_void_p


class gdp_problem(ctypes.Structure):
    _fields_ = [("L", ctypes.c_int32), ("V", ctypes.c_int32), ("S", ctypes.c_int32),
                ("mem", _ptr), ("intra", _ptr), ("inter", _ptr), ("inter_index", _ptr),
                ("n_inter", ctypes.c_int32), ("n_key", ctypes.c_int32),
                ("other_mem", _ptr), ("other_time", _ptr), ("flags", ctypes.c_uint32), ("f0", _ptr)]


class gdp_result(ctypes.Structure):
    _fields_ = [("total", _ptr), ("remaining", _ptr), ("res", _ptr), ("f_out", _ptr), ("mark_out", _ptr)]


class gdp_timing(ctypes.Structure):
    _fields_ = [("total_ms", ctypes.c_float), ("relax_ms", ctypes.c_float), ("relax_launches", ctypes.c_int32),
                ("fused", ctypes.c_int32), ("relaxations", ctypes.c_double), ("executed", ctypes.c_double),
                ("relax_bytes", ctypes.c_double), ("tile_ts", ctypes.c_int32), ("tile_r", ctypes.c_int32),
                ("keep_marks", ctypes.c_int32), ("chunk", ctypes.c_int32),
                ("latency_variant", ctypes.c_int32), ("flow", ctypes.c_int32), ("fused_split", ctypes.c_int32)]


class gdp_batch_stats(ctypes.Structure):
    _fields_ = [("relaxations", ctypes.c_double), ("executed", ctypes.c_double), ("device_ms", ctypes.c_double),
                ("instances", ctypes.c_int64), ("parts", ctypes.c_int64), ("flow_parts", ctypes.c_int64),
                ("fused_parts", ctypes.c_int64), ("per_layer_parts", ctypes.c_int64)]


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python __graft_entry__.py` "
                               "(galvatron_dp._build.build()); there is no CPU fallback")
        L = ctypes.CDLL(LIB_PATH)
        pp = ctypes.POINTER(ctypes.POINTER(gdp_problem))
        rp = ctypes.POINTER(ctypes.POINTER(gdp_result))
        L.gdp_solve.argtypes = [ctypes.POINTER(gdp_problem), ctypes.POINTER(gdp_result)]
        L.gdp_solve.restype = ctypes.c_int
        L.gdp_solve_static.argtypes = [ctypes.POINTER(gdp_problem), ctypes.POINTER(gdp_result)]
        L.gdp_solve_static.restype = ctypes.c_int
        L.gdp_solve_batch.argtypes = [ctypes.c_int32, pp, rp]
        L.gdp_solve_batch.restype = ctypes.c_int
        L.gdp_plan_create.argtypes = [ctypes.c_int32, pp, ctypes.POINTER(ctypes.c_void_p)]
        L.gdp_plan_create.restype = ctypes.c_int
        L.gdp_plan_run.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.POINTER(gdp_timing)]
        L.gdp_plan_run.restype = ctypes.c_int
        L.gdp_plan_fetch.argtypes = [ctypes.c_void_p, rp]
        L.gdp_plan_fetch.restype = ctypes.c_int
        L.gdp_plan_set_option.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64]
        L.gdp_plan_set_option.restype = ctypes.c_int
        L.gdp_plan_destroy.argtypes = [ctypes.c_void_p]
        L.gdp_plan_destroy.restype = None
        L.gdp_cache_trim.argtypes = []
        L.gdp_cache_trim.restype = None
        L.gdp_last_error.argtypes = []
        L.gdp_last_error.restype = ctypes.c_char_p
        L.gdp_version.argtypes = []
        L.gdp_version.restype = ctypes.c_int
        L.gdp_device_info.argtypes = [ctypes.c_char_p, ctypes.c_size_t]
        L.gdp_device_info.restype = ctypes.c_int
        L.gdp_debug_check_layout.argtypes = [ctypes.c_int32, pp, ctypes.c_int32, ctypes.c_int64]
        L.gdp_debug_check_layout.restype = ctypes.c_int
        L.gdp_debug_shared_device.argtypes = [ctypes.c_int32]
        L.gdp_debug_shared_device.restype = None
        L.gdp_batch_stats_begin.argtypes = []
        L.gdp_batch_stats_begin.restype = None
        L.gdp_batch_stats_end.argtypes = [ctypes.POINTER(gdp_batch_stats)]
        L.gdp_batch_stats_end.restype = ctypes.c_int
        _lib = L
    return _lib


def _check(rc: int) -> None:
    if rc == GDP_OK:
        return
    msg = lib().gdp_last_error().decode("utf-8", "replace")
    if rc == GDP_E_UNSUPPORTED:
        raise UnsupportedInputError(msg)
    if rc in (GDP_E_BADARG, GDP_E_NONFINITE):
        raise ValueError(msg)
    if rc == GDP_E_NOMEM:
        raise MemoryError(msg)
    raise RuntimeError(f"galvatron_dp_hip error {rc}: {msg}")


def device_info() -> str:
    buf = ctypes.create_string_buffer(256)
    _check(lib().gdp_device_info(buf, 256))
    return buf.value.decode()


_from_buffer = ctypes.c_char.from_buffer
_addressof = ctypes.addressof


def _addr(a):
    """Address of a C-contiguous array's data (None for None).  Through the buffer protocol where the array
    allows it: a quarter of the time of building ``__array_interface__``, and a search makes thousands of
    problems."""
    if a is None:
        return None
    try:
        return _addressof(_from_buffer(a))
    except (TypeError, ValueError):            # read-only or empty
        return a.__array_interface__['data'][0]


class Problem:
    """One DP instance (the arguments of one reference plugin call) with host arrays in the
    dtypes/layouts the C ABI wants, plus the output arrays it will fill."""

    def __init__(self, mem, intra, inter, V: int, other_mem: Sequence[int], other_time: Sequence[float], *,
                 inter_index=None, export_f: bool = False, export_mark: bool = False, launch: str | None = None,
                 compute_all: bool = False, keep_marks: bool = False, f0=None):
        self.mem = np.ascontiguousarray(mem, dtype=np.int32)
        if self.mem.ndim != 2:
            raise ValueError("mem must be [L,S]")
        self.L, self.S = self.mem.shape
        self.V = int(V)
        self.intra = np.ascontiguousarray(intra, dtype=np.float64)
        self.inter = np.ascontiguousarray(inter, dtype=np.float64)
        if self.intra.shape != (self.L, self.S):
            raise ValueError("intra must be [L,S]")
        if self.inter.ndim != 3 or self.inter.shape[1:] != (self.S, self.S):
            raise ValueError("inter must be [T,S,S]")
        if inter_index is None:
            if self.inter.shape[0] != self.L:
                raise ValueError("inter must be [L,S,S] when inter_index is not given")
            self.inter_index = None
        else:
            self.inter_index = np.ascontiguousarray(inter_index, dtype=np.int32)
            if self.inter_index.shape != (self.L,):
                raise ValueError("inter_index must be [L]")
        self.other_mem = np.ascontiguousarray(other_mem, dtype=np.int64).reshape(-1)
        self.other_time = np.ascontiguousarray(other_time, dtype=np.float64).reshape(-1)
        if self.other_mem.shape != self.other_time.shape:
            raise ValueError("other_mem and other_time must have one entry per key")
        self.n_key = int(self.other_mem.shape[0])
        # initial costs [V,S] (what the reference's caller leaves in ``_f``); the library treats zeros as None
        self.f0 = None
        if f0 is not None:
            self.f0 = np.ascontiguousarray(f0, dtype=np.float64)
            if self.f0.size != self.V * self.S:
                raise ValueError("f0 must be [V,S]")
        if launch not in (None, "fused", "per_layer"):
            raise ValueError("launch must be None, 'fused' or 'per_layer'")
        self.flags = ((GDP_EXPORT_F if export_f else 0) | (GDP_EXPORT_MARK if export_mark else 0) |
                      (GDP_LAUNCH_FUSED if launch == "fused" else 0) |
                      (GDP_LAUNCH_PER_LAYER if launch == "per_layer" else 0) |
                      (GDP_COMPUTE_ALL if compute_all else 0) | (GDP_KEEP_MARKS if keep_marks else 0))
        if self.V < 1 or self.L < 1 or self.S < 1:
            raise ValueError("L, V and S must be >= 1")
        # outputs
        self.total = np.empty(self.n_key, dtype=np.float64)
        self.total.fill(np.inf)
        self.remaining = np.empty(self.n_key, dtype=np.int32)
        self.remaining.fill(-1)
        self.res = np.empty((self.n_key, self.L), dtype=np.int32)
        self.res.fill(-1)
        self.f_out = np.empty((self.V, self.S), dtype=np.float64) if export_f else None
        self.mark_out = np.empty((self.L, self.V, self.S), dtype=np.int32) if export_mark else None
        addr = _addr
        self._c_problem = gdp_problem(
            self.L, self.V, self.S, addr(self.mem), addr(self.intra), addr(self.inter), addr(self.inter_index),
            int(self.inter.shape[0]), self.n_key, addr(self.other_mem), addr(self.other_time), self.flags,
            addr(self.f0))
        self._c_result = gdp_result(addr(self.total), addr(self.remaining), addr(self.res), addr(self.f_out),
                                    addr(self.mark_out))

    @property
    def relaxations(self) -> int:
        return self.L * self.V * self.S * self.S


def _arrays(problems: Sequence[Problem]):
    n = len(problems)
    P = (ctypes.POINTER(gdp_problem) * n)(*[ctypes.pointer(p._c_problem) for p in problems])
    R = (ctypes.POINTER(gdp_result) * n)(*[ctypes.pointer(p._c_result) for p in problems])
    return P, R


def cache_trim() -> None:
    """gdp_cache_trim: frees the device allocations that finished plans left behind for reuse."""
    lib().gdp_cache_trim()


def solve_batch(problems: Sequence[Problem]) -> None:
    """gdp_solve_batch: fills ``total``/``remaining``/``res`` (and exports) of every problem."""
    if not problems:
        return
    P, R = _arrays(problems)
    _check(lib().gdp_solve_batch(len(problems), P, R))


def check_layout(problems: Sequence[Problem], num_cu: int = 256, lds_per_cu: int = 160 * 1024) -> None:
    """gdp_debug_check_layout: lays the plan out for a described device (no device needed) and checks
    every address the kernels would form; raises with the violated bound."""
    P, _ = _arrays(problems)
    _check(lib().gdp_debug_check_layout(len(problems), P, num_cu, lds_per_cu))


def debug_shared_device(seems_shared: bool) -> None:
    """gdp_debug_shared_device: puts the library into (or takes it out of) the state it enters when a waiting
    launch was given up: launches that never wait are then chosen wherever the choice is the library's."""
    lib().gdp_debug_shared_device(1 if seems_shared else 0)


def batch_stats_begin() -> None:
    """gdp_batch_stats_begin: start adding up what the process's gdp_solve_batch calls do."""
    lib().gdp_batch_stats_begin()


def batch_stats_end() -> gdp_batch_stats:
    """gdp_batch_stats_end: stop, and return the sums (relaxations, device time of the parts, ...)."""
    s = gdp_batch_stats()
    _check(lib().gdp_batch_stats_end(ctypes.byref(s)))
    return s


def solve_static(problem: Problem) -> None:
    """gdp_solve_static: one instance, solved in the library's static device array (no allocation)."""
    _check(lib().gdp_solve_static(ctypes.byref(problem._c_problem), ctypes.byref(problem._c_result)))


class Plan:
    """gdp_plan_*: inputs resident on the device, the device part runnable repeatedly."""

    def __init__(self, problems: Sequence[Problem]):
        self.problems = list(problems)
        self._P, self._R = _arrays(self.problems)
        h = ctypes.c_void_p()
        _check(lib().gdp_plan_create(len(self.problems), self._P, ctypes.byref(h)))
        self._h = h

    def set_option(self, option: int, value: int) -> None:
        _check(lib().gdp_plan_set_option(self._h, option, value))

    def run(self, timing_mode: int = 0) -> gdp_timing:
        t = gdp_timing()
        _check(lib().gdp_plan_run(self._h, timing_mode, ctypes.byref(t)))
        return t

    def fetch(self) -> None:
        _check(lib().gdp_plan_fetch(self._h, self._R))

    def close(self) -> None:
        if self._h is not None and self._h.value:
            lib().gdp_plan_destroy(self._h)
        self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
