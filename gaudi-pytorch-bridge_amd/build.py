"""Builds the two shared libraries of the package, in-tree.

  libmi355q.so     gfx950 HIP kernels behind the C ABI of include/mi355q.h
                   (hipcc, no torch dependency)
  mi355q_torch.so  TORCH_LIBRARY(hpu) host layer that calls the C ABI
                   (g++ against the installed PyTorch-ROCm)
  libmi355q_probe.so  measurement probes (csrc/bench/), loaded by
                   ``bench.py --only ceilings`` alone; not part of the product ABI

Run as ``python gaudi-pytorch-bridge_amd/build.py`` or call ``build()``.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB_KERNELS = os.path.join(HERE, "libmi355q.so")
LIB_TORCH = os.path.join(HERE, "mi355q_torch.so")
LIB_PROBE = os.path.join(HERE, "libmi355q_probe.so")

HIP_SOURCES = ["cast_kernels.hip", "int4_kernels.hip", "reduce_kernels.hip", "gemm_api.hip", "gemm_inst_kk.hip", "gemm_inst_km.hip", "gemm_inst_mk.hip", "gemm_inst_mm.hip", "w4_gemm.hip", "sdpa_kernels.hip", "api.cpp"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 VALU ops are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option", "-Wno-inline-asm",
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        sys.stderr.write(r.stdout)
        raise RuntimeError("build step failed: " + " ".join(cmd))
    if verbose and r.stdout.strip():
        lines = [l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l]
        if lines:
            print("\n".join(lines), flush=True)


def build_kernels(verbose=False, jobs=8):
    os.makedirs(OBJ, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    cmds = []
    for src in HIP_SOURCES:
        obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
        objs.append(obj)
        cmds.append([hipcc] + HIPCC_FLAGS + ["-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj])
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(lambda c: _run(c, verbose), cmds))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_KERNELS] + objs, verbose)
    return LIB_KERNELS


def build_probes(verbose=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    _run([hipcc] + HIPCC_FLAGS + ["-shared", "-x", "hip", os.path.join(CSRC, "bench", "probe_kernels.hip"), "-o", LIB_PROBE], verbose)
    return LIB_PROBE


def build_torch_ext(verbose=False):
    import torch
    from torch.utils import cpp_extension as ce
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = []
    for p in ce.include_paths():
        inc += ["-isystem", p]
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-Wall", "-Wno-unused-function", "-Wno-deprecated-declarations"] + inc + \
          ["-isystem", os.path.join(rocm, "include"),
           os.path.join(CSRC, "torch_ops.cpp"), "-o", LIB_TORCH,
           "-L" + tlib, "-lc10", "-ltorch_cpu", "-ltorch", "-lc10_hip", "-ltorch_hip",
           "-L" + HERE, "-lmi355q", "-Wl,-rpath,$ORIGIN", "-Wl,--no-as-needed"]
    _run(cmd, verbose)
    return LIB_TORCH


def build(verbose=False, jobs=8):
    with ThreadPoolExecutor(max_workers=2) as ex:
        k = ex.submit(build_kernels, verbose, jobs)
        p = ex.submit(build_probes, verbose)
        k.result()
        p.result()
    build_torch_ext(verbose)
    return LIB_KERNELS, LIB_TORCH


if __name__ == "__main__":
    build(verbose=True)
    print("built", LIB_KERNELS, LIB_TORCH)
