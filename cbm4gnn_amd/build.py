"""Build the two shared libraries of the package in-tree.

    libcbm_hip.so   hipcc, gfx950 only: the HIP kernels and their C-ABI launchers
    libcbm_host.so  g++ / OpenMP: the host-side format builder

Run ``python -m cbm4gnn_amd.build`` (no GPU needed: hipcc cross-compiles).  The reference builds
its extension with cmake + setuptools against MKL and arbok (``cbm/setup.py:15-47``); none of
that applies here.
"""
from __future__ import annotations

import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
SRC_DIR = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
HIP_LIB = os.path.join(LIB_DIR, "libcbm_hip.so")
HOST_LIB = os.path.join(LIB_DIR, "libcbm_host.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

HIP_FLAGS = [
    "-O3", "--offload-arch=gfx950", "-shared", "-fPIC", "-std=c++17",
    "-ffp-contract=off",                       # FMAs are written explicitly where they are meant
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
HOST_FLAGS = ["-O3", "-fopenmp", "-shared", "-fPIC", "-std=c++17", "-Wall"]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops' is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"build failed ({proc.returncode}): {' '.join(cmd)}\n{out}")
    return out


def build_hip(verbose: bool = False) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    out = _run([HIPCC, *HIP_FLAGS, "-o", HIP_LIB, os.path.join(SRC_DIR, "cbm_kernels.hip")])
    if verbose and out.strip():
        print(out)
    return HIP_LIB


def build_host(verbose: bool = False) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    out = _run(["g++", *HOST_FLAGS, "-o", HOST_LIB, os.path.join(SRC_DIR, "cbm_builder.cpp")])
    if verbose and out.strip():
        print(out)
    return HOST_LIB


def build_all(verbose: bool = False):
    return build_hip(verbose), build_host(verbose)


if __name__ == "__main__":
    for p in build_all(verbose=True):
        print("built", p)
    sys.exit(0)
