"""Compiles the HIP sources in ../csrc into ../lib/libgalvatron_dp_hip.so for gfx950.

hipcc cross-compiles without a GPU, so this runs in any ROCm container.  The built library is
kept in-tree (git-ignored) and is what ``galvatron_dp._lib`` loads.
"""
from __future__ import annotations

import os
import subprocess

PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(PKG, "csrc")
LIB_DIR = os.path.join(PKG, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libgalvatron_dp_hip.so")
SOURCES = ["gdp_kernels.hip", "gdp_api.hip", "gdp_static.hip"]
ARCH = "gfx950"
# -ffp-contract=off: the recurrence has no multiply, but nothing may ever be fused or reassociated.
# packed-fp32-ops is switched off for every HIP translation unit built here.
HIPCC_FLAGS = ["-O3", "-std=c++17", f"--offload-arch={ARCH}", "-fPIC", "-shared", "-ffp-contract=off",
               "-fno-fast-math", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall",
               "-Wno-unused-command-line-argument"]


def build(verbose: bool = False, extra_flags=(), out: str = LIB_PATH, csrc: str = CSRC) -> str:
    os.makedirs(os.path.dirname(out), exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + HIPCC_FLAGS + list(extra_flags) + [os.path.join(csrc, s) for s in SOURCES] + ["-o", out]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = "\n".join(l for l in proc.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + log)
    if verbose and log.strip():
        print(log)
    return out


if __name__ == "__main__":
    print(build(verbose=True))
