"""Builds libeuler_hip.so (HIP kernels + C-ABI + the C++ euler:: API) for gfx950 with hipcc.

    python deep-learning-math-kernel-research_amd/build.py

The library is written next to this file so that it travels with the source tree.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libeuler_hip.so")

SOURCES = [
    "ehip_gemm.hip",
    "ehip_gemm1x1.hip",
    "ehip_gemm1x1w.hip",
    "ehip_conv3x3v.hip",
    "ehip_fewch.hip",
    "ehip_depthwise.hip",
    "ehip_wino.hip",
    "ehip_wino_lanes.hip",
    "ehip_prepare.hip",
    "ehip_harness.hip",
    "ehip_api.hip",
    "euler_api.hip",
]

# -ffp-contract=off: every single-rounding multiply-add of the reference is written as an explicit
#   fma; nothing else may fuse, or float results stop being bit-identical.
# packed-fp32-ops off: keep the compiler from forming packed fp32 instructions.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


# per-source additions.  The depthwise matrix-core kernel has one accumulator tile per wave and turns it
# straight into bytes: in the accumulation registers every value would be moved in and out once.
EXTRA_FLAGS = {
    "ehip_depthwise.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1", "-mllvm", "-amdgpu-kernarg-preload-count=16"],
    # the 3x3 kernel takes what its first instructions need as leading scalar arguments: preloaded with the wave
    # (and its straight-line K loops are 72 steps of ~250 instructions: beyond the default budget of
    # `#pragma unroll`, which then leaves a loop whose weight registers are indexed at run time, i.e. in scratch)
    "ehip_conv3x3v.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=16", "-mllvm", "-pragma-unroll-threshold=1000000"],
    # the resident-tile 1x1 kernel's leading scalar arguments: preloaded as well
    "ehip_gemm1x1.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=16"],
    # the Winograd kernel whose requantized values take the accumulators' place in the vector registers
    "ehip_wino_lanes.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "ehip_gemm1x1w.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=16", "-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    # and those of the 1x1 kernels with few input channels
    "ehip_gemm.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=16"],
}


def _stale(obj, src):
    """an object is reused only when it is newer than its source and every header"""
    if not os.path.exists(obj):
        return True
    deps = [src] + [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")] + \
        [os.path.join(ROOT, "include", f) for f in os.listdir(os.path.join(ROOT, "include"))] + [__file__]
    return any(os.path.getmtime(d) > os.path.getmtime(obj) for d in deps)


def build(verbose=True, jobs=8, incremental=False):
    """incremental: recompile only what changed (development); the default compiles everything"""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    objs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src + ".o")
        objs.append(obj)
        if incremental and not _stale(obj, os.path.join(CSRC, src)):
            continue
        cmd = [hipcc] + FLAGS + EXTRA_FLAGS.get(src, []) + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        if len(procs) >= jobs:
            _wait(procs)
    _wait(procs)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    # the MFMA rate probe of the benchmark: a library of its own, not part of the product's C-ABI
    cmd = [hipcc] + FLAGS + ["-shared", os.path.join(CSRC, "ehip_probe.hip"), "-o", os.path.join(objdir, "libehip_probe.so")]
    if verbose:
        print(" ".join(cmd), flush=True)
    procs.append(("ehip_probe.hip", subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
    _wait(procs)
    # a small client of the C++ API (include/euler.hpp), used by the GPU tests
    check = os.path.join(objdir, "euler_api_check")
    cmd = [hipcc, "-O2", "-std=c++17", "-I" + os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "cxx", "euler_api_check.cpp"), "-o", check,
           "-L" + HERE, "-leuler_hip", "-Wl,-rpath," + HERE, "-Wl,-rpath,$ORIGIN/.."]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    # every reorder<> instantiation behind one C entry point, used by the CPU tests (host code only)
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-shared", "-fPIC", "-I" + os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "cxx", "reorder_check.cpp"), "-o", os.path.join(objdir, "libreorder_check.so"),
           "-L" + HERE, "-leuler_hip", "-Wl,-rpath," + HERE, "-Wl,-rpath,$ORIGIN/.."]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


def _wait(procs):
    failed = []
    for src, p in procs:
        out, _ = p.communicate()
        text = out.decode(errors="replace")
        # the host pass does not know the packed-fp32 feature name; that warning is harmless
        text = "\n".join(l for l in text.splitlines() if "packed-fp32-ops" not in l)
        if text.strip():
            print(text)
        if p.returncode != 0:
            failed.append(src)
    procs.clear()
    if failed:
        raise RuntimeError("hipcc failed for: " + ", ".join(failed))


if __name__ == "__main__":
    build(incremental="--incremental" in sys.argv)
    print("built", LIB)
