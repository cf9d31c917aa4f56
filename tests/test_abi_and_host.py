"""CPU-only checks of the boundary: the shared library loads, exports every symbol the header
declares, and the host-side argument handling behaves (no compute call is made here)."""
import ctypes
import os
import re

import numpy as np
import pytest

from galvatron_dp import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "galvatron_dp_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gdp_[a-z_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    lib = _lib.lib()
    names = _declared_symbols()
    assert set(names) == set(_lib.EXPORTED_SYMBOLS), names
    for n in names:
        assert getattr(lib, n) is not None


def test_version_and_struct_sizes():
    assert _lib.lib().gdp_version() == 102
    assert ctypes.sizeof(_lib.gdp_problem) == 88
    assert ctypes.sizeof(_lib.gdp_result) == 40
    assert ctypes.sizeof(_lib.gdp_timing) == 72


def test_validation_happens_before_any_device_work():
    # these are rejected on the host, so they behave the same with or without a GPU
    lib = _lib.lib()
    mem = np.ones((2, 3), np.int32)
    intra = np.ones((2, 3))
    inter = np.zeros((2, 3, 3))

    def rc_of(p):
        h = ctypes.c_void_p()
        P = (ctypes.POINTER(_lib.gdp_problem) * 1)(ctypes.pointer(p._c_problem))
        return lib.gdp_plan_create(1, P, ctypes.byref(h)), lib.gdp_last_error().decode()

    mn = mem.copy(); mn[0, 0] = -3
    assert rc_of(_lib.Problem(mn, intra, inter, 10, [0], [0.0]))[0] == _lib.GDP_E_BADARG
    bad = intra.copy(); bad[0, 2] = np.nan
    assert rc_of(_lib.Problem(mem, bad, inter, 10, [0], [0.0]))[0] == _lib.GDP_E_NONFINITE
    bad = inter.copy(); bad[1, 2, 0] = -np.inf
    assert rc_of(_lib.Problem(mem, intra, bad, 10, [0], [0.0]))[0] == _lib.GDP_E_NONFINITE
    huge = intra.copy(); huge[:] = 1e300
    assert rc_of(_lib.Problem(mem, huge, inter, 10, [0], [0.0]))[0] == _lib.GDP_E_NONFINITE
    big_s = np.ones((1, _lib.GDP_MAX_S + 1), np.int32)
    p = _lib.Problem(big_s, np.ones((1, _lib.GDP_MAX_S + 1)), np.zeros((1, _lib.GDP_MAX_S + 1, _lib.GDP_MAX_S + 1)),
                     10, [0], [0.0])
    assert rc_of(p)[0] == _lib.GDP_E_BADARG
    n = _lib.GDP_MAX_S_MARKS + 1      # the argmin table has byte entries: no table above 256 strategies
    p = _lib.Problem(np.ones((1, n), np.int32), np.ones((1, n)), np.zeros((1, n, n)), 10, [0], [0.0], export_mark=True)
    assert rc_of(p)[0] == _lib.GDP_E_BADARG
    p = _lib.Problem(np.ones((1, n), np.int32), np.ones((1, n)), np.zeros((1, n, n)), 10, [0], [0.0], keep_marks=True)
    assert rc_of(p)[0] == _lib.GDP_E_BADARG
    assert lib.gdp_plan_create(0, None, ctypes.byref(ctypes.c_void_p())) == _lib.GDP_E_BADARG
    # a negative other_mem would put the start row V-1-other_mem above the table (the reference reads out of
    # bounds there, csrc/dp_core.cpp:82-89); one above V-1 is merely an infeasible key and is accepted
    rc, msg = rc_of(_lib.Problem(mem, intra, inter, 10, [0, -1], [0.0, 0.0]))
    assert rc == _lib.GDP_E_BADARG and "other_mem" in msg
    rc, msg = rc_of(_lib.Problem(mem, intra, inter, 10, [-(1 << 40)], [0.0]))
    assert rc == _lib.GDP_E_BADARG and "other_mem" in msg
    too_tall = _lib.Problem(mem, intra, inter, (1 << 30) + 1, [0], [0.0])
    assert rc_of(too_tall)[0] == _lib.GDP_E_BADARG
    # the initial costs (what the reference's caller leaves in _f): NaN and -inf like in the cost arrays, and
    # no negative zero; zeros and +inf are fine (checked with the layout audit, which needs no device)
    f0 = np.ones((10, 3))
    for bad_value, code in ((np.nan, _lib.GDP_E_NONFINITE), (-np.inf, _lib.GDP_E_NONFINITE), (-0.0, _lib.GDP_E_BADARG),
                            (1e300, _lib.GDP_E_NONFINITE)):
        g = f0.copy(); g[7, 1] = bad_value
        rc, msg = rc_of(_lib.Problem(mem, intra, inter, 10, [0], [0.0], f0=g))
        assert rc == code and ("f0" in msg or "overflow" in msg), (bad_value, rc, msg)
    with pytest.raises(ValueError):
        _lib.Problem(mem, intra, inter, 10, [0], [0.0], f0=np.ones((9, 3)))
    ok = f0.copy(); ok[2, 2] = np.inf
    _lib.check_layout([_lib.Problem(mem, intra, inter, 10, [0], [0.0], f0=ok)])
    _lib.check_layout([_lib.Problem(mem, intra, inter, 10, [0], [0.0], f0=np.zeros((10, 3)))])


def test_static_entry_point_refuses_on_the_host():
    """gdp_solve_static checks the arguments and the size of its fixed working memory before it touches
    the device: an instance that does not fit is refused with both sizes in the message."""
    lib = _lib.lib()
    S, L, V = 44, 32, 65536                          # the argmin table alone is 92 MB
    p = _lib.Problem(np.ones((L, S), np.int32), np.ones((L, S)), np.zeros((1, S, S)), V, [0], [0.0],
                     inter_index=np.zeros(L, np.int32))
    rc = lib.gdp_solve_static(ctypes.byref(p._c_problem), ctypes.byref(p._c_result))
    msg = lib.gdp_last_error().decode()
    assert rc == _lib.GDP_E_NOMEM and str(_lib.GDP_STATIC_SCRATCH_BYTES) in msg and "gdp_solve" in msg, msg
    with pytest.raises(MemoryError):
        _lib.solve_static(p)
    mem = np.ones((2, 3), np.int32)
    q = _lib.Problem(mem, np.ones((2, 3)), np.zeros((2, 3, 3)), 10, [0], [0.0], export_f=True)
    assert lib.gdp_solve_static(ctypes.byref(q._c_problem), ctypes.byref(q._c_result)) == _lib.GDP_E_BADARG
    q = _lib.Problem(mem, np.ones((2, 3)), np.zeros((2, 3, 3)), 10, [-2], [0.0])
    assert lib.gdp_solve_static(ctypes.byref(q._c_problem), ctypes.byref(q._c_result)) == _lib.GDP_E_BADARG
    assert lib.gdp_solve_static(None, None) == _lib.GDP_E_BADARG


def test_problem_shape_checks():
    with pytest.raises(ValueError):
        _lib.Problem(np.ones((2, 3), np.int32), np.ones((2, 4)), np.zeros((2, 3, 3)), 10, [0], [0.0])
    with pytest.raises(ValueError):
        _lib.Problem(np.ones((2, 3), np.int32), np.ones((2, 3)), np.zeros((1, 3, 3)), 10, [0], [0.0])
    with pytest.raises(ValueError):
        _lib.Problem(np.ones((2, 3), np.int32), np.ones((2, 3)), np.zeros((2, 3, 3)), 10, [0, 1], [0.0])
    p = _lib.Problem(np.ones((2, 3), np.int32), np.ones((2, 3)), np.zeros((1, 3, 3)), 10, [0], [0.0],
                     inter_index=[0, 0])
    assert p.relaxations == 2 * 10 * 9


def test_problem_points_at_the_arrays_it_keeps():
    """The C structure of a problem holds the addresses of the arrays the Python object keeps alive --
    also for arrays that do not allow a writable view (read-only inputs) and for key lists of length
    zero, where the address comes from another route."""
    mem = np.arange(6, dtype=np.int32).reshape(2, 3) + 1
    intra = np.ones((2, 3))
    inter = np.zeros((2, 3, 3))
    for a in (mem, intra, inter):
        a.setflags(write=False)
    p = _lib.Problem(mem, intra, inter, 10, [0, 3], [0.0, 1.0])
    c = p._c_problem
    addr = lambda a: a.__array_interface__["data"][0]      # noqa: E731
    assert (c.mem, c.intra, c.inter) == (addr(p.mem), addr(p.intra), addr(p.inter))
    assert p.mem is mem and p.intra is intra and p.inter is inter      # no copies of arrays that already fit
    assert (c.other_mem, c.other_time) == (addr(p.other_mem), addr(p.other_time))
    r = p._c_result
    assert (r.total, r.remaining, r.res) == (addr(p.total), addr(p.remaining), addr(p.res))
    assert list(p.total) == [np.inf, np.inf] and list(p.remaining) == [-1, -1] and (p.res == -1).all()
    q = _lib.Problem(mem.copy(), intra.copy(), inter.copy(), 10, [], [])
    assert q.n_key == 0 and q.total.shape == (0,)


def test_static_entry_point_links_against_nothing_that_allocates(tmp_path):
    """gdp_solve_static exists for callers that may not obtain memory.  Its translation unit is compiled
    alone and its undefined symbols are looked through: no device, page-locked or host allocator, no stream
    or event creation; and of the library's other translation units only helpers that allocate nothing
    (validation, error text, kernel launchers)."""
    import shutil
    import subprocess
    from galvatron_dp import _build
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if shutil.which(hipcc) is None:
        pytest.skip("no hipcc")
    obj = str(tmp_path / "gdp_static.o")
    flags = [f for f in _build.HIPCC_FLAGS if f != "-shared"]
    proc = subprocess.run([hipcc] + flags + ["-c", os.path.join(_build.CSRC, "gdp_static.hip"), "-o", obj],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout[-2000:]
    undefined = subprocess.run(["nm", "-u", "-C", obj], stdout=subprocess.PIPE, text=True, check=True).stdout
    names = [ln.split(None, 1)[1].strip() for ln in undefined.splitlines() if ln.strip().startswith("U ")]
    assert any(n.startswith("hipGetSymbolAddress") for n in names), names
    forbidden = ("hipMalloc", "hipHostMalloc", "hipExtMalloc", "hipHostAlloc", "hipMemAlloc", "hipStreamCreate",
                 "hipEventCreate", "hipFree", "hipHostFree", "operator new", "operator delete", "malloc", "calloc",
                 "realloc", "posix_memalign", "aligned_alloc", "std::__throw_length_error", "std::__throw_bad_alloc")
    for n in names:
        assert not any(n == f or n.startswith(f + "(") or n.startswith(f + "[") or (f.startswith("hip") and n.startswith(f))
                       for f in forbidden), f"gdp_static.hip refers to {n}"
    allowed_own = {"gdp_clear_error", "gdp_fail", "gdp_fail_hip", "gdp_validate", "gdp_validate_f0", "gdp_find_variant",
                   "gdp_launch_init", "gdp_launch_relax", "gdp_launch_zero_pass", "gdp_launch_epilogue"}
    own = {n.split("(")[0] for n in names if n.startswith("gdp_")}
    assert own <= allowed_own, own - allowed_own


def test_export_switch_is_per_thread():
    """The reference's parallel search calls the plugin from many threads: a thread that asks for ``_f`` /
    ``_mark`` to be written back must not change what the other threads allocate and copy."""
    import threading

    import galvatron_dp_core as shim
    seen = {}

    def worker():
        seen["before"] = shim.export_enabled()
        shim.set_export(True)
        seen["after"] = shim.export_enabled()

    assert shim.export_enabled() is False
    t = threading.Thread(target=worker)
    t.start()
    t.join()
    assert seen == {"before": False, "after": True}
    assert shim.export_enabled() is False
    shim.set_export(True)
    try:
        assert shim.export_enabled() is True
    finally:
        shim.set_export(False)
