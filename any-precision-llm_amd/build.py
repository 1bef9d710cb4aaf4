"""Builds the in-tree native libraries of this package.

    python build.py            # libanyprec_hip.so (hipcc, gfx950) + host-check lib (g++)

The HIP library is cross-compiled; no GPU is needed to build it.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")

HIP_LIB = os.path.join(LIBDIR, "libanyprec_hip.so")
HOSTCHECK_LIB = os.path.join(LIBDIR, "libanyprec_hostcheck.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fno-gpu-rdc",
    "-Wall", "-Wno-unused-function",
]


def _hipcc() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found")


def build_hip(verbose: bool = False, extra_flags=()) -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra_flags, "-I", INCLUDE, "-I", CSRC,
           os.path.join(CSRC, "ap_capi.hip"), "-o", HIP_LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the packed-fp32 feature and says so; drop that line
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return HIP_LIB


def build_hostcheck(verbose: bool = False) -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unknown-pragmas", "-I", CSRC,
           os.path.join(CSRC, "ap_hostcheck.cpp"), "-o", HOSTCHECK_LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return HOSTCHECK_LIB


def build_all(verbose: bool = False) -> None:
    build_hip(verbose)
    build_hostcheck(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
    print("built:", HIP_LIB, HOSTCHECK_LIB)
