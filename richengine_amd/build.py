"""Builds libkvx.so (HIP kernels + C ABI) for gfx950, in-tree."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libkvx.so")
SOURCES = ["kvx_host.cpp", "kvx_pool.cpp", "kvx_pool_abi.cpp", "kvx_prefix.cpp",
           "kvx_prefix_abi.cpp", "kvx_kernels.hip",
           "kvx_decode_int4.hip", "kvx_attend_wide.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall",
         # packed fp32 instructions stay off for every kernel of this library
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-I", os.path.join(ROOT, "include"), "-I", CSRC]


def build(verbose=True, lib=LIB, extra_flags=(), tag=""):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objects = []
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    for src in SOURCES:
        obj = os.path.join(HERE, "build", src + tag + ".o")
        cmd = [hipcc, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj] + FLAGS + list(extra_flags)
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
        objects.append(obj)
    cmd = [hipcc, "-shared", "-o", lib] + objects + ["--offload-arch=gfx950"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return lib


HOST_TEST_SRC = os.path.join(ROOT, "tests", "cpp", "kvx_host_test.cpp")
HOST_TEST_BIN = os.path.join(ROOT, "tests", "cpp", "kvx_host_test")


def build_host_test(verbose=True):
    """The C++ test of the host mirror (include/kvx.hpp): host code only, linked
    against libkvx.so and the HIP runtime."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, "-x", "c++", "-std=c++17", "-O1", "-Wall", "-D__HIP_PLATFORM_AMD__",
           "-I", os.path.join(ROOT, "include"), "-I", "/opt/rocm/include", HOST_TEST_SRC,
           "-o", HOST_TEST_BIN, "-L", HERE, "-lkvx", "-L", "/opt/rocm/lib", "-lamdhip64",
           "-Wl,-rpath,$ORIGIN/../../richengine_amd"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return HOST_TEST_BIN


if __name__ == "__main__":
    build()
    build_host_test()
    print(LIB)
