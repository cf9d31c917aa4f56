"""The CPU-side code under AddressSanitizer + UndefinedBehaviorSanitizer (no GPU involved): the C
restatement of the reference's DP, and the host side of the HIP library -- argument validation and
the whole plan layout, whose every derived address is then audited (gdp_debug_check_layout).  The
programs live in tests/sanitize/; they are compiled here with the sanitizer run-times linked
statically and run as child processes, which exit non-zero on any finding."""
import os
import shutil
import subprocess

import numpy as np
import pytest

from galvatron_dp import _build, _lib, workloads as W

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SRC = os.path.join(HERE, "sanitize")
OUT = os.path.join(SRC, "_build")
ENV = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1")


def _run(cmd, **kw):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, **kw)
    lines = [ln for ln in proc.stdout.splitlines() if "is not a recognized feature for this target" not in ln]
    assert proc.returncode == 0, "\n".join([" ".join(cmd)] + lines[-40:])
    return lines


def test_oracle_under_sanitizers():
    os.makedirs(OUT, exist_ok=True)
    exe = os.path.join(OUT, "oracle_check")
    _run(["gcc", "-O1", "-g", "-std=c11", "-ffp-contract=off", "-fsanitize=address,undefined",
          "-fno-sanitize-recover=all", "-static-libasan", os.path.join(SRC, "oracle_check.c"), "-lm", "-o", exe])
    out = _run([exe], env=ENV)
    assert any("cases clean" in ln for ln in out), out


@pytest.mark.skipif(shutil.which(os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")) is None, reason="no hipcc")
def test_library_host_code_under_sanitizers():
    """Instruments the host pass only (each -fsanitize right after -Xarch_host); the device pass is
    compiled as for the shipped library."""
    os.makedirs(OUT, exist_ok=True)
    exe = os.path.join(OUT, "host_check")
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    flags = [f for f in _build.HIPCC_FLAGS if f not in ("-O3", "-shared", "-fPIC")]
    _run([hipcc, "-O1", "-g"] + flags +
         ["-Xarch_host", "-fsanitize=address,undefined", "-Xarch_host", "-fno-sanitize-recover=all", "-static-libsan",
          os.path.join(SRC, "host_check.cpp")] + [os.path.join(_build.CSRC, s) for s in _build.SOURCES] + ["-o", exe])
    symbols = subprocess.run(["nm", exe], stdout=subprocess.PIPE, text=True).stdout
    assert "__asan_init" in symbols and "__ubsan_handle" in symbols, "the host pass was not instrumented"
    out = _run([exe], env=ENV)
    assert any("layouts audited" in ln for ln in out), out


def test_layout_audit_through_the_library():
    """The same audit through the shipped (uninstrumented) library, on the five benchmark shapes and a
    few odd ones; an input that validation rejects never reaches the layout."""
    def prob(inst, **kw):
        keys = sorted(inst.other_mem)
        return _lib.Problem(inst.mem, inst.intra, inst.inter_tables if inst.inter_tables is not None else inst.inter,
                            inst.V, [inst.other_mem[k] for k in keys], [inst.other_time[k] for k in keys],
                            inter_index=inst.inter_index, **kw)
    for cfg in (0, 1, 2, 4):
        _lib.check_layout([prob(W.CONFIGS[cfg]())])
        _lib.check_layout([prob(W.CONFIGS[cfg](), keep_marks=True)], num_cu=304, lds_per_cu=64 * 1024)
    _lib.check_layout([prob(i) for i in W.config3(n_limit=48)])
    rng = np.random.Generator(np.random.PCG64(3))
    odd = [W.random_instance(rng, L, S, V, mem_hi=max(1, V // 3)) for (L, S, V) in
           [(1, 1, 1), (2, 1, 2), (3, 1024, 64), (9, 257, 333), (40, 3, 100001)]]
    for inst in odd:
        _lib.check_layout([prob(inst)])
    # a dense [L,S,S] array that repeats matrices (they are kept once): runs of equal ones, one that comes
    # back later, and more different ones than the library looks back at
    inst = W.random_instance(rng, 24, 5, 300, mem_hi=40)
    dense = inst.inter[[0, 0, 1, 1, 0, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 11, 3, 10, 0, 12, 12, 12, 1, 13]]
    keys = sorted(inst.other_mem)
    _lib.check_layout([_lib.Problem(inst.mem, inst.intra, np.ascontiguousarray(dense), inst.V,
                                    [inst.other_mem[k] for k in keys], [inst.other_time[k] for k in keys])])
    bad = W.random_instance(rng, 3, 4, 50, mem_hi=9)
    with pytest.raises(ValueError):                       # validation comes first: a start row above the table
        _lib.check_layout([_lib.Problem(bad.mem, bad.intra, bad.inter, bad.V, [-1], [0.0])])
