"""Compiles the HIP sources of this package into lib/liblitenn_hip.so for gfx950."""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "liblitenn_hip.so")
# the same library with the streaming GEMV's timeline stamps compiled in, plus the measurement
# kernels of csrc/microbench.hip; only bench.py --microbench loads it
TRACE_LIB_PATH = os.path.join(LIB_DIR, "liblitenn_hip_trace.so")

SOURCES = ["api.hip", "gemv.hip", "gemm.hip", "glue.hip", "attn_tile.hip", "primitives.hip", "llama.hip", "gguf.hip"]
# gemv.hip: the dispatcher hands the first six kernel arguments over in registers (the streaming
# kernel's activation pointer, K and first-row addressing), see gemv_stream_kernel
# glue.hip: the attention step's pointers, among them the device-resident position it loads first
SOURCE_FLAGS = {"gemv.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=6"],
                "glue.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=6"]}

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # packed-FP32 instruction selection is switched off for every device function
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP backend cannot be built")
    return exe


def build(verbose: bool = True, jobs: int = 6) -> str:
    """Compile every source (always, even if a library is already present) and link."""
    os.makedirs(LIB_DIR, exist_ok=True)
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    procs, objs = [], []
    trace_units = [("gemv.hip", "gemv_trace.o", ["-DLITENN_GEMV_TRACE"]), ("microbench.hip", "microbench.o", [])]
    for src, obj_name, extra in [(s, s.replace(".hip", ".o"), []) for s in SOURCES] + trace_units:
        obj = os.path.join(obj_dir, obj_name)
        if not extra and src in SOURCES:
            objs.append(obj)
        cmd = [hipcc(), *HIPCC_FLAGS, *SOURCE_FLAGS.get(src, []), *extra, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        while sum(p.poll() is None for _, p in procs) >= jobs:
            procs[0][1].wait()
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if p.returncode != 0:
            failed = True
            print(f"--- {src} failed ---\n{out}", file=sys.stderr)
        elif verbose and out:
            print(out)
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc",
           "-Wl,--version-script=" + os.path.join(CSRC, "exports.map"), *objs, "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    trace_objs = [os.path.join(obj_dir, "gemv_trace.o") if o.endswith(os.sep + "gemv.o") else o for o in objs]
    trace_objs.append(os.path.join(obj_dir, "microbench.o"))
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc",
           "-Wl,--version-script=" + os.path.join(CSRC, "exports.map"), *trace_objs, "-o", TRACE_LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB_PATH


CPP_TEST_SRC = os.path.join(os.path.dirname(HERE), "tests", "cpp", "device_traits_test.cpp")
CPP_TEST_BIN = os.path.join(os.path.dirname(HERE), "tests", "cpp", "device_traits_test")


def build_cpp_host_test(verbose: bool = True) -> str:
    """Compile the C++ host-side test of include/LiteNN/Device/HIP.h against the built library
    (plain g++, C++20; no GPU code in it)."""
    cxx = shutil.which("g++") or shutil.which("c++")
    if not cxx:
        raise RuntimeError("g++ not found; the C++ host test cannot be built")
    cmd = [cxx, "-std=c++20", "-O1", "-Wall", "-I", os.path.join(os.path.dirname(HERE), "include"), CPP_TEST_SRC,
           "-L", LIB_DIR, "-llitenn_hip", "-Wl,-rpath,$ORIGIN/../../litenn_amd/lib", "-o", CPP_TEST_BIN]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return CPP_TEST_BIN


FETCH_TEST_SRC = os.path.join(os.path.dirname(HERE), "tests", "cpp", "fetch_bounds_test.cpp")
FETCH_TEST_BIN = os.path.join(os.path.dirname(HERE), "tests", "cpp", "fetch_bounds_test")


def build_fetch_bounds_test(verbose: bool = True) -> str:
    """Compile the host-side bounds model of the kernels' fetch patterns (plain g++: it includes
    csrc/fetch_model.hpp, the address arithmetic the kernels themselves call)."""
    cxx = shutil.which("g++") or shutil.which("c++")
    if not cxx:
        raise RuntimeError("g++ not found; the fetch bounds test cannot be built")
    cmd = [cxx, "-std=c++17", "-O2", "-Wall", FETCH_TEST_SRC, "-o", FETCH_TEST_BIN]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return FETCH_TEST_BIN


if __name__ == "__main__":
    build()
    build_cpp_host_test()
    build_fetch_bounds_test()
