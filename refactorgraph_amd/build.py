"""Builds the native libraries in-tree (refactorgraph_amd/lib/):

    librg_hip.so     HIP kernels + C ABI (include/rg_hip.h), gfx950 only
    librg_host.so    C++ host layer mirroring the reference's plugin surface
                     (hardware::Device, runtime::Resources/Routine, kernel::Kernel,
                     collectors); links librg_hip.so
    librg_probe.so   measurement aids of bench.py (bench_probes/): ceilings of the matrix pipe
                     and of HBM; not part of the boundary, loaded by the benchmark only

hipcc cross-compiles for gfx950 without a GPU, so this runs anywhere the ROCm toolchain is
installed.  Usage: ``python -m refactorgraph_amd.build [--jobs N]``.
"""
from __future__ import annotations

import argparse
import concurrent.futures as cf
import glob
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
HOST = os.path.join(PKG, "host")
LIB = os.path.join(PKG, "lib")
OBJ = os.path.join(LIB, "obj")
INCLUDE = os.path.join(ROOT, "include")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

# packed-fp32 VALU ops are switched off for all device code (target feature, device pass only)
HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++20", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    f"-I{INCLUDE}", f"-I{CSRC}",
]
HOST_FLAGS = ["-O2", "-std=c++20", "-fPIC", "-Wall", "-Wextra", f"-I{INCLUDE}", f"-I{os.path.join(HOST, 'include')}"]


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + proc.stdout + proc.stderr)
        raise RuntimeError(f"build step failed: {cmd[0]} {cmd[-1]}")
    # the host pass of hipcc warns that it does not know the packed-fp32 feature: harmless
    return proc


def _compile_hip(src):
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    _run([HIPCC, *HIP_FLAGS, "-c", src, "-o", obj])
    return obj


def _compile_host(src):
    obj = os.path.join(OBJ, "host_" + os.path.basename(src) + ".o")
    _run(["g++", *HOST_FLAGS, "-c", src, "-o", obj])
    return obj


def build_hip(jobs=8):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile_hip, srcs))
    out = os.path.join(LIB, "librg_hip.so")
    _run([HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", out])
    return out


def build_host(jobs=8):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(HOST, "src", "*.cc")))
    if not srcs:
        return None
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile_host, srcs))
    out = os.path.join(LIB, "librg_host.so")
    _run(["g++", "-shared", "-fPIC", *objs, "-o", out, f"-L{LIB}", "-lrg_hip", "-Wl,-rpath,$ORIGIN"])
    return out


def build_probes():
    os.makedirs(OBJ, exist_ok=True)
    out = os.path.join(LIB, "librg_probe.so")
    _run([HIPCC, *HIP_FLAGS, "-shared", os.path.join(PKG, "bench_probes", "probes.hip"), "-o", out])
    return out


def build_all(jobs=8):
    hip = build_hip(jobs)
    host = build_host(jobs)
    probes = build_probes()
    return hip, host, probes


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=8)
    args = ap.parse_args()
    for path in build_all(args.jobs):
        if path:
            print("built", os.path.relpath(path, ROOT))
