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
OBJDIR = os.path.join(HERE, "build")
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


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the packed-fp32 feature and says so; drop that line
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + out)
    if verbose and out.strip():
        print(out)


def build_hip(verbose: bool = False, extra_flags=(), jobs: int = 8) -> str:
    """One object per kernel family and bit-width (compiled in parallel) + the C ABI, linked into the .so."""
    from concurrent.futures import ThreadPoolExecutor

    os.makedirs(OBJDIR, exist_ok=True)
    os.makedirs(LIBDIR, exist_ok=True)
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"] + list(extra_flags) + ["-I", INCLUDE, "-I", CSRC, "-c"]
    units = [(os.path.join(CSRC, "ap_capi.hip"), os.path.join(OBJDIR, "ap_capi.o"), [])]
    for b in range(3, 9):
        units.append((os.path.join(CSRC, "ap_gemv_inst.hip"), os.path.join(OBJDIR, f"ap_gemv_b{b}.o"), [f"-DAP_BITS={b}"]))
        units.append((os.path.join(CSRC, "ap_gemvf_inst.hip"), os.path.join(OBJDIR, f"ap_gemvf_b{b}.o"), [f"-DAP_BITS={b}"]))
        units.append((os.path.join(CSRC, "ap_gemvp_inst.hip"), os.path.join(OBJDIR, f"ap_gemvp_b{b}.o"), [f"-DAP_BITS={b}"]))
        units.append((os.path.join(CSRC, "ap_gemm_inst.hip"), os.path.join(OBJDIR, f"ap_gemm_b{b}.o"), [f"-DAP_BITS={b}"]))
        units.append((os.path.join(CSRC, "ap_gemmw_inst.hip"), os.path.join(OBJDIR, f"ap_gemmw_b{b}.o"), [f"-DAP_BITS={b}"]))
        units.append((os.path.join(CSRC, "ap_gemmt_inst.hip"), os.path.join(OBJDIR, f"ap_gemmt_b{b}.o"), [f"-DAP_BITS={b}"]))
        units.append((os.path.join(CSRC, "ap_gemv4_inst.hip"), os.path.join(OBJDIR, f"ap_gemv4_b{b}.o"), [f"-DAP_BITS={b}"]))
    hipcc = _hipcc()
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(lambda u: _run([hipcc, *compile_flags, *u[2], u[0], "-o", u[1]], verbose), units))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *[u[1] for u in units], "-o", HIP_LIB],
         verbose)
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
