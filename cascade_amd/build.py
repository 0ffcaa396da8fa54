"""Compiles the native libraries of this package in-tree.

  libcascade_hip.so        hand-written HIP for gfx950 behind the C ABI of include/cascade_hip.h
  libcascade_workloads.so  host-only generator of the synthetic benchmark partitions
  cascade_sa               the reference's command-line builder (text file in, sa40 file out) over the C ABI

Run as `python -m cascade_amd.build`. hipcc cross-compiles for gfx950 without a GPU.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
HIP_LIB = os.path.join(HERE, "libcascade_hip.so")
WORKLOADS_LIB = os.path.join(HERE, "libcascade_workloads.so")
CLI = os.path.join(HERE, "cascade_sa")

HIPCC_FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-shared", "-Wall",
    # packed FP32 instructions stay off (nothing here is floating point, the flag is policy for this target)
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # machine-level loop-invariant code motion hoists values out of loops that then stay live through the whole body:
    # without it partition_ids_kernel fits 5 waves per SIMD instead of 4 (8.7 -> 7.7 ms per 1e9 suffixes); the other
    # kernels are unchanged by it
    "-mllvm", "-disable-machine-licm",
]


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def build_hip(extra_flags=()):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    _run([hipcc, *HIPCC_FLAGS, *extra_flags, "-o", HIP_LIB, os.path.join(CSRC, "cascade_hip.hip")])
    return HIP_LIB


def build_workloads():
    cc = os.environ.get("CC", "gcc")
    _run([cc, "-std=c11", "-O2", "-fopenmp", "-fPIC", "-shared", "-Wall", "-Wextra", "-o", WORKLOADS_LIB,
          os.path.join(CSRC, "workloads.c"), "-lm"])
    return WORKLOADS_LIB


def build_cli():
    """The host-side mirror of the reference's builder (include/cascade_gpu_saca.hpp) as a program: plain g++, linked
    against libcascade_hip.so next to it."""
    cxx = os.environ.get("CXX", "g++")
    _run([cxx, "-std=c++17", "-O2", "-Wall", "-Wextra", "-Werror", "-o", CLI, os.path.join(CSRC, "cascade_sa.cpp"),
          "-L" + HERE, "-lcascade_hip", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath-link,/opt/rocm/lib"])
    return CLI


def build_cpp_tests():
    """tests/cpp/slab_pipeline: a multi-partition build through the slab members of include/cascade_gpu_saca.hpp, in the
    reference's own language (the GPU suite runs it). Host code; needs the HIP runtime only for its own device buffers."""
    cxx = os.environ.get("CXX", "g++")
    root = os.path.dirname(HERE)
    out = os.path.join(root, "tests", "cpp", "slab_pipeline")
    _run([cxx, "-std=c++17", "-O2", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__", "-isystem", "/opt/rocm/include", "-o", out,
          os.path.join(root, "tests", "cpp", "slab_pipeline.cpp"), "-L" + HERE, "-lcascade_hip", "-L/opt/rocm/lib", "-lamdhip64",
          "-Wl,-rpath,$ORIGIN/../../cascade_amd", "-Wl,-rpath,/opt/rocm/lib", "-pthread"])
    return out


def build_all():
    build_hip()
    build_workloads()
    build_cli()
    build_cpp_tests()


if __name__ == "__main__":
    build_all()
    sys.exit(0)
