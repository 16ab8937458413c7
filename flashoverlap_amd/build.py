"""Builds the two native libraries in-tree, for gfx950 only.

  flashoverlap_amd/lib/libfo_hip.so        HIP kernels + the C ABI (hipcc)
  flashoverlap_amd/lib/libst_pybinding.so  OverlapImpl / BaselineImpl / ops (g++ + torch headers),
                                           linked against libfo_hip.so only through the C ABI
  flashoverlap_amd/lib/libfo_bench.so      measurement probes that only bench.py and its test load
                                           (include/flashoverlap_bench.h); not part of the product

Usage: python -m flashoverlap_amd.build [--only hip|binding|bench] [-j N]
hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is.
"""
from __future__ import annotations

import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "lib")
OBJ = os.path.join(HERE, "build")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

HIP_SOURCES = ["fo_capi.hip", "fo_gemm.hip", "fo_sync.hip", "fo_rmsnorm.hip", "fo_static.hip"]
BENCH_SOURCES = ["fo_probe.hip"]
BINDING_SOURCES = ["overlap_impl.cpp", "baseline_impl.cpp", "rmsnorm_op.cpp", "pybind.cpp"]

# -packed-fp32-ops: keep hipcc from forming packed-fp32 instructions out of scalar float code.
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-command-line-argument"]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in proc.stdout.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError("build step failed: " + " ".join(cmd) + "\n" + out)
    if out.strip():
        print(out)


def _build_hip_library(sources, name: str, jobs: int) -> str:
    os.makedirs(LIB, exist_ok=True)
    os.makedirs(OBJ, exist_ok=True)
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    objs = [os.path.join(OBJ, s.replace(".hip", ".o")) for s in sources]
    cmds = [[hipcc, *HIPCC_FLAGS, "-c", os.path.join(CSRC, s), "-o", o] for s, o in zip(sources, objs)]
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(_run, cmds))
    out = os.path.join(LIB, name)
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", out])
    return out


def build_hip(jobs: int = 4) -> str:
    return _build_hip_library(HIP_SOURCES, "libfo_hip.so", jobs)


def build_bench(jobs: int = 4) -> str:
    return _build_hip_library(BENCH_SOURCES, "libfo_bench.so", jobs)


def build_binding(jobs: int = 4) -> str:
    import torch
    from torch.utils import cpp_extension as ext

    os.makedirs(LIB, exist_ok=True)
    os.makedirs(OBJ, exist_ok=True)
    inc = [f"-I{p}" for p in ext.include_paths()] + [f"-I{ROCM}/include", f"-I{os.path.join(HERE, '..', 'include')}"]
    flags = ["-O2", "-fPIC", "-std=c++17", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
             f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-Wno-deprecated-declarations"]
    objs = [os.path.join(OBJ, s.replace(".cpp", ".o")) for s in BINDING_SOURCES]
    cmds = [["g++", *flags, *inc, "-c", os.path.join(CSRC, s), "-o", o] for s, o in zip(BINDING_SOURCES, objs)]
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(_run, cmds))
    tlib = ext.library_paths()[0]
    out = os.path.join(LIB, "libst_pybinding.so")
    _run(["g++", "-shared", "-fPIC", *objs, "-o", out,
          f"-L{LIB}", "-lfo_hip", f"-L{tlib}", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch",
          "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tlib}"])
    return out


def build_all(jobs: int = 4) -> None:
    build_hip(jobs)
    build_binding(jobs)
    build_bench(jobs)


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--only", choices=["hip", "binding", "bench"])
    ap.add_argument("-j", type=int, default=4)
    a = ap.parse_args()
    if a.only in (None, "hip"):
        print(build_hip(a.j))
    if a.only in (None, "binding"):
        print(build_binding(a.j))
    if a.only in (None, "bench"):
        print(build_bench(a.j))
    sys.exit(0)
