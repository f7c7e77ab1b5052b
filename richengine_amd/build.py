"""Builds libkvx.so (HIP kernels + C ABI) for gfx950, in-tree."""
import concurrent.futures
import json
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libkvx.so")
SOURCES = ["kvx_host.cpp", "kvx_pool.cpp", "kvx_pool_abi.cpp", "kvx_prefix.cpp",
           "kvx_prefix_abi.cpp", "kvx_kernels.hip",
           "kvx_decode_int4.hip", "kvx_attend_wide.hip", "kvx_calibrate.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall",
         # packed fp32 instructions stay off for every kernel of this library
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         # no fused multiply-adds but the ones the sources spell out (fmaf): the oracle is built the
         # same way, and a product fused into the difference behind it turns a score minus the
         # maximum it equals into the product's rounding error (__fmul_rn and its like are plain
         # operators in HIP's headers and fuse like any other, whatever pragma surrounds the call)
         "-ffp-contract=off",
         "-I", os.path.join(ROOT, "include"), "-I", CSRC]
# What the compiler reports per kernel (registers, scratch bytes per lane, spills,
# waves per SIMD) goes to this file next to the library, so that a change that
# sends a hot kernel to scratch memory shows up without a GPU.
RESOURCES = os.path.join(HERE, "kernel_resources.json")
REMARK = re.compile(r"remark:\s+(Function Name|VGPRs|AGPRs|ScratchSize \[bytes/lane\]|"
                    r"Occupancy \[waves/SIMD\]|VGPRs Spill|LDS Size \[bytes/block\]): (\S+)")


def kernel_resources(compiler_stderr):
    """{kernel name: {field: value}} from -Rpass-analysis=kernel-resource-usage remarks."""
    kernels, current = {}, None
    for line in compiler_stderr.splitlines():
        m = REMARK.search(line)
        if not m:
            continue
        field, value = m.groups()
        if field == "Function Name":
            current = kernels.setdefault(value, {})
        elif current is not None:
            current[field.split(" [")[0].replace(" ", "_").lower()] = int(value)
    return kernels


def build(verbose=True, lib=LIB, extra_flags=(), tag=""):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objects, resources = [], {}
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    def compile_one(src):
        obj = os.path.join(HERE, "build", src + tag + ".o")
        cmd = [hipcc, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj] + FLAGS + list(extra_flags)
        if src.endswith(".hip"):
            cmd.append("-Rpass-analysis=kernel-resource-usage")
        if verbose:
            print(" ".join(cmd), flush=True)
        return obj, cmd, subprocess.run(cmd, stderr=subprocess.PIPE, text=True)

    # the sources compile side by side (the kernel files take most of the time), and their
    # remarks are read in the order of SOURCES
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as pool:
        compiled = list(pool.map(compile_one, SOURCES))
    for obj, cmd, done in compiled:
        # the remarks and the host pass's note about the packed-fp32 feature are not warnings
        for line in done.stderr.splitlines():
            if "kernel-resource-usage" in line or "packed-fp32-ops" in line:
                continue
            if re.match(r"\s*\d* *\||\s*\^|In file included from", line) and "warning" not in done.stderr:
                continue
            print(line, file=sys.stderr)
        if done.returncode:
            raise subprocess.CalledProcessError(done.returncode, cmd)
        resources.update(kernel_resources(done.stderr))
        objects.append(obj)
    cmd = [hipcc, "-shared", "-o", lib] + objects + ["--offload-arch=gfx950"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    if lib == LIB:
        with open(RESOURCES, "w") as out:
            json.dump(resources, out, indent=1, sort_keys=True)
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
