"""Builds the gfx950 binaries in-tree (hipcc cross-compiles without a GPU):

  libwhirl_sampling_hip.so   the C-ABI library (include/whirl_sampling_abi.h)
  whirl_sampling_gfx950.co   the code object alone, for callers that resolve kernels by name (hipModuleGetFunction)
  libwhirl_sampling_host.so  the C++ host API (include/sampling/*.h, include/whirl/*.h) over the C-ABI library

Usage: python whirl-llm_amd/build.py
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "csrc", "ws_abi.hip")
SRC_FUSED = os.path.join(HERE, "csrc", "ws_fused.hip")  # the single-sweep sampler kernel
SRC_SPLIT = os.path.join(HERE, "csrc", "ws_split.hip")  # the same kernel for rows split over several workgroups
SRC_KEPT = [os.path.join(HERE, "csrc", f) for f in ("ws_fused_kept.hip", "ws_split_kept.hip")]  # both once more, with the kept-set dump
SRC_SHORT = os.path.join(HERE, "csrc", "ws_short.hip")  # the short-list kernel for batches whose rows all have a bounded top-k
SRC_LEAN = os.path.join(HERE, "csrc", "ws_lean.hip")  # the lean single-sweep kernel for batches of unsplit rows
# packed FP32 instructions are switched off for every device compile of this repository
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         # the fused sweep is one fully unrolled loop of ~20 batches (its bin cache must stay in registers)
         "-mllvm", "-pragma-unroll-threshold=262144"]


def run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "'-packed-fp32-ops' is not a recognized feature"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError("build failed: " + " ".join(cmd) + "\n" + err)
    return err


HOST_SRCS = [os.path.join(HERE, "host", f) for f in ("sampler.cpp", "acceptor.cpp", "spec_sample.cpp", "device_rows.cpp", "host_c_api.cpp")]
INCLUDE = os.path.join(os.path.dirname(HERE), "include")


def build(verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    so = os.path.join(HERE, "libwhirl_sampling_hip.so")
    co = os.path.join(HERE, "whirl_sampling_gfx950.co")
    host = os.path.join(HERE, "libwhirl_sampling_host.so")
    # the five translation units and the bare code object side by side (each takes a minute or two), then the link
    objdir = os.path.join(HERE, "csrc", "obj")
    os.makedirs(objdir, exist_ok=True)
    srcs = (SRC, SRC_FUSED, SRC_SPLIT, *SRC_KEPT, SRC_LEAN, SRC_SHORT)
    objs = [os.path.join(objdir, os.path.basename(src)[:-4] + ".o") for src in srcs]
    jobs = [[hipcc, *FLAGS, "-fPIC", "-c", "-o", obj, src] for obj, src in zip(objs, srcs)]
    jobs.append([hipcc, *FLAGS, "--genco", "-o", co, SRC])
    with concurrent.futures.ThreadPoolExecutor(max_workers=8) as pool:
        list(pool.map(run, jobs))
    run([hipcc, "--offload-arch=gfx950", "-fPIC", "-shared", "-o", so, *objs])
    # host layer: plain C++20, no device code; -ffp-contract=off keeps the float arithmetic of the penalties unfused
    run([os.environ.get("CXX", "g++"), "-std=c++20", "-O2", "-fPIC", "-shared", "-ffp-contract=off", "-Wall", "-Wextra",
         "-D__HIP_PLATFORM_AMD__", "-I" + INCLUDE, "-I" + os.path.join(rocm, "include"), "-o", host, *HOST_SRCS,
         "-L" + HERE, "-lwhirl_sampling_hip", "-L" + os.path.join(rocm, "lib"), "-lamdhip64", "-Wl,-rpath,$ORIGIN",
         "-Wl,-rpath," + os.path.join(rocm, "lib")])
    if verbose:
        print("built", so, "and", co, "and", host)
    return so, co


if __name__ == "__main__":
    build()
    sys.exit(0)
