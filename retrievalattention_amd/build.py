"""Builds libretro_mi355.so (HIP kernels + host wave buffer) for gfx950 with hipcc.

    python -m retrievalattention_amd.build

The library is written next to this file so that it travels with the source tree.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libretro_mi355.so")
HIP_SOURCES = ["capi.hip", "score.hip", "select.hip", "attend.hip", "gather.hip", "kmeans.hip", "lru.hip"]
CPP_SOURCES = ["wavebuf.cpp"]
ARCH = "gfx950"
# -ffp-contract=off: products and sums round separately unless the source says fmaf, which
# keeps the k-means reductions reproducible on a CPU.  The packed-fp32 feature is disabled
# because some of its instruction forms have been unreliable on this hardware pool.
HIP_FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-ffp-contract=off",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]
# per-file additions: the k-means assignment reads every MFMA accumulator in its argmax
# epilogue, so its accumulators live in ordinary VGPRs (no accumulator-register copies)
EXTRA_HIP_FLAGS = {"kmeans.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}
CPP_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-pthread"]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("build step failed: " + " ".join(cmd) + "\n" + r.stdout)
    return r.stdout


def build(verbose=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    jobs = []
    for s in HIP_SOURCES:
        o = os.path.join(objdir, s + ".o")
        jobs.append(([hipcc] + HIP_FLAGS + EXTRA_HIP_FLAGS.get(s, []) + ["-c", os.path.join(CSRC, s), "-o", o], o))
    for s in CPP_SOURCES:
        o = os.path.join(objdir, s + ".o")
        jobs.append(([hipcc] + CPP_FLAGS + ["-c", os.path.join(CSRC, s), "-o", o], o))
    with ThreadPoolExecutor(max_workers=min(6, len(jobs))) as ex:
        outs = list(ex.map(lambda j: _run(j[0]), jobs))
    if verbose:
        for o in outs:
            if o.strip():
                print(o)
    objs = [j[1] for j in jobs]
    _run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", LIB] + objs + ["-pthread"])
    build_capi_example(hipcc)
    return LIB


# A plain HIP program that drives a decode step through the C ABI (no Python, no torch); tests/test_gpu_capi.py
# runs it.  It finds the library next to the package through its run path.
CAPI_EXAMPLE_SRC = os.path.join(os.path.dirname(HERE), "tests", "capi_decode_step.cpp")
CAPI_EXAMPLE = os.path.join(os.path.dirname(HERE), "tests", "capi_decode_step")


def build_capi_example(hipcc):
    if not os.path.exists(CAPI_EXAMPLE_SRC):
        return None
    _run([hipcc, "-O2", "-std=c++17", f"--offload-arch={ARCH}", "-I", os.path.join(os.path.dirname(HERE), "include"),
          CAPI_EXAMPLE_SRC, "-o", CAPI_EXAMPLE, "-L", HERE, "-l:libretro_mi355.so",
          "-Wl,-rpath,$ORIGIN/../retrievalattention_amd"])
    return CAPI_EXAMPLE


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
