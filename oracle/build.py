"""Build recipe for the CPU checkers (test infrastructure only).

* ``build_oracle()``  compiles ``oracle/dp_oracle.c`` (the plain-C restatement)
  into ``oracle/libdp_oracle.so``.
* ``build_ref()``     compiles the reference's own translation unit,
  ``/root/reference/csrc/dp_core.cpp``, from where it lies, with the flags of the
  reference's recipe (``Makefile:1-16``: ``g++ -O3 -Wall -shared -std=c++11 -fPIC``
  plus the pybind11 include paths), into ``oracle/_ref/``.  No reference source is
  copied; only the built extension module lands in ``oracle/_ref`` (git-ignored).
  It is skipped when ``/root/reference`` is not present (e.g. on a GPU box, which
  only uses the prebuilt file).

Nothing in the shipped library imports this module.
"""
from __future__ import annotations

import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "libdp_oracle.so")
REF_DIR = os.path.join(HERE, "_ref")
REF_SRC = "/root/reference/csrc/dp_core.cpp"
REF_MODULE = "galvatron_dp_core"


def ref_so_path() -> str:
    return os.path.join(REF_DIR, REF_MODULE + sysconfig.get_config_var("EXT_SUFFIX"))


def build_oracle(verbose: bool = False) -> str:
    cmd = ["gcc", "-O3", "-std=c11", "-fPIC", "-shared", "-ffp-contract=off",
           "-fno-fast-math", "-Wall", "-Wextra",
           os.path.join(HERE, "dp_oracle.c"), "-o", ORACLE_SO, "-lm"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return ORACLE_SO


def build_ref(verbose: bool = False) -> str | None:
    if not os.path.exists(REF_SRC):
        return None
    import pybind11

    os.makedirs(REF_DIR, exist_ok=True)
    out = ref_so_path()
    cmd = ["g++", "-O3", "-Wall", "-shared", "-std=c++11", "-fPIC",
           "-I" + pybind11.get_include(), "-I" + sysconfig.get_paths()["include"],
           REF_SRC, "-o", out]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return out


if __name__ == "__main__":
    print(build_oracle(verbose=True))
    print(build_ref(verbose=True))
    sys.exit(0)
