"""Builds the two native libraries in-tree:

  libgrouped_gemm_hip.so            HIP kernels + C ABI (hipcc, gfx950 only)
  grouped_gemm_backend.<abi>.so     PyTorch-ROCm binding (g++, links the first)

Usage: python grouped_gemm_amd/build.py [--force]
hipcc cross-compiles gfx950 without a GPU, so this runs anywhere the ROCm toolchain
and PyTorch-ROCm are installed.
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
ROOT = os.path.dirname(HERE)
HIP_LIB = os.path.join(HERE, "libgrouped_gemm_hip.so")
EXT_LIB = os.path.join(HERE, "grouped_gemm_backend" + sysconfig.get_config_var("EXT_SUFFIX"))

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC", "-shared",
    # packed fp32 instructions are switched off for device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _newer(target, sources):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(s) <= t for s in sources)


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l)
    if res.returncode != 0:
        raise RuntimeError("build step failed:\n" + out)
    if out.strip():
        print(out)


def build_hip(force=False):
    sources = [os.path.join(CSRC, f) for f in ("gmm_api.hip", "gmm_kernel.hpp")]
    sources.append(os.path.join(ROOT, "include", "grouped_gemm_hip.h"))
    if not force and _newer(HIP_LIB, sources):
        return HIP_LIB
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    _run([hipcc] + HIPCC_FLAGS + [os.path.join(CSRC, "gmm_api.hip"), "-o", HIP_LIB])
    return HIP_LIB


def build_binding(force=False):
    import torch
    src = os.path.join(CSRC, "torch_binding.cpp")
    if not force and _newer(EXT_LIB, [src, HIP_LIB, os.path.join(ROOT, "include", "grouped_gemm_hip.h")]):
        return EXT_LIB
    tdir = os.path.dirname(torch.__file__)
    tlib = os.path.join(tdir, "lib")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = [
        os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=grouped_gemm_backend",
        "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
        "-I" + os.path.join(tdir, "include"),
        "-I" + os.path.join(tdir, "include", "torch", "csrc", "api", "include"),
        "-I" + os.path.join(rocm, "include"),
        "-I" + sysconfig.get_paths()["include"],
        src, "-o", EXT_LIB,
        "-L" + HERE, "-lgrouped_gemm_hip",
        "-L" + tlib, "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10", "-lc10_hip", "-ltorch_hip",
        "-L" + os.path.join(rocm, "lib"), "-lamdhip64",
        "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + tlib, "-Wl,-rpath," + os.path.join(rocm, "lib"),
    ]
    _run(cmd)
    return EXT_LIB


def build_all(force=False):
    build_hip(force)
    build_binding(force)
    return HIP_LIB, EXT_LIB


if __name__ == "__main__":
    build_all(force="--force" in sys.argv)
