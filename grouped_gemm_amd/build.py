"""Builds the two native libraries in-tree:

  libgrouped_gemm_hip.so            HIP kernels + C ABI (hipcc, gfx950 only)
  grouped_gemm_backend.<abi>.so     PyTorch-ROCm binding (g++, links the first)

Usage: python grouped_gemm_amd/build.py [--force]
hipcc cross-compiles gfx950 without a GPU, so this runs anywhere the ROCm toolchain
and PyTorch-ROCm are installed.  The kernel variants (csrc/gmm_variants.def) are compiled as
separate translation units, several at a time; objects are kept under grouped_gemm_amd/build/.

build_bench_probe() builds bench.py's own helper (bench_mfma_probe.hip at the repository root,
a matrix-instruction rate probe) into libbench_mfma_probe.so next to it; it is no part of the
library.
"""
import os
import re
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
ROOT = os.path.dirname(HERE)
HIP_LIB = os.path.join(HERE, "libgrouped_gemm_hip.so")
EXT_LIB = os.path.join(HERE, "grouped_gemm_backend" + sysconfig.get_config_var("EXT_SUFFIX"))

OBJ_DIR = os.path.join(HERE, "build")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC",
    # packed fp32 instructions are switched off for device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # the asm that loads into LDS names m0 as clobbered; clang notes that m0 is a reserved register
    "-Wno-inline-asm",
]


def _newer(target, sources):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(s) <= t for s in sources)


def _run(cmd, quiet=False):
    if not quiet:
        print("+", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l)
    if res.returncode != 0:
        raise RuntimeError("build step failed: " + " ".join(cmd) + "\n" + out)
    if out.strip():
        print(out)


def variant_indices():
    """Indices listed in csrc/gmm_variants.def: one translation unit per kernel variant."""
    text = open(os.path.join(CSRC, "gmm_variants.def")).read()
    return [int(m) for m in re.findall(r"^GG_VARIANT\((\d+),", text, flags=re.M)]


def build_hip(force=False, jobs=None):
    headers = [os.path.join(CSRC, f) for f in ("gmm_kernel.hpp", "gmm_generic.hpp", "gmm_variants.hpp",
                                               "gmm_variants.def")]
    headers.append(os.path.join(ROOT, "include", "grouped_gemm_hip.h"))
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    obj_dir, hip_lib, extra = OBJ_DIR, HIP_LIB, []
    os.makedirs(obj_dir, exist_ok=True)
    units = [(os.path.join(CSRC, "gmm_api.hip"), os.path.join(obj_dir, "gmm_api.o"), extra)]
    for i in variant_indices():
        units.append((os.path.join(CSRC, "gmm_variant.hip"), os.path.join(obj_dir, f"gmm_variant_{i}.o"),
                      extra + [f"-DGG_VARIANT_INDEX={i}"]))
    for dt in range(4):   # gmm_generic.hpp, one translation unit per element type
        units.append((os.path.join(CSRC, "gmm_generic_variant.hip"), os.path.join(obj_dir, f"gmm_generic_{dt}.o"),
                      extra + [f"-DGG_GENERIC_DT={dt}"]))
    todo = [u for u in units if force or not _newer(u[1], [u[0]] + headers)]
    jobs = jobs or min(len(todo) or 1, int(os.environ.get("MAX_JOBS", os.cpu_count() or 1)))
    if todo:
        print(f"compiling {len(todo)} translation units with {hipcc}, {jobs} at a time", flush=True)
        with ThreadPoolExecutor(max_workers=jobs) as pool:
            list(pool.map(lambda u: _run([hipcc] + HIPCC_FLAGS + u[2] + ["-c", u[0], "-o", u[1]], quiet=True), todo))
    objects = [u[1] for u in units]
    if todo or not _newer(hip_lib, objects):
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objects + ["-o", hip_lib])
    return hip_lib


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


BENCH_PROBE_SRC = os.path.join(ROOT, "bench_mfma_probe.hip")
BENCH_PROBE_LIB = os.path.join(ROOT, "libbench_mfma_probe.so")


def build_bench_probe(force=False):
    """bench.py's helper: the rate of the bf16 matrix instruction alone (not part of the library)."""
    if not force and _newer(BENCH_PROBE_LIB, [BENCH_PROBE_SRC]):
        return BENCH_PROBE_LIB
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    _run([hipcc] + HIPCC_FLAGS + ["-shared", BENCH_PROBE_SRC, "-o", BENCH_PROBE_LIB])
    return BENCH_PROBE_LIB


def build_all(force=False):
    build_hip(force)
    build_binding(force)
    build_bench_probe(force)
    return HIP_LIB, EXT_LIB


if __name__ == "__main__":
    build_all(force="--force" in sys.argv)
