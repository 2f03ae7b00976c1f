"""Builds libpfeife_hip.so (gfx950 only) in-tree with hipcc.

    python -m pfeife_amd.hip.build          # compile every source, link the library

The library is written next to this file so that it travels with the source
tree; nothing is installed.  hipcc cross-compiles gfx950 code objects without a
GPU present.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.normpath(os.path.join(HERE, "..", "csrc"))
LIB_PATH = os.path.join(HERE, "libpfeife_hip.so")
OBJ_DIR = os.path.join(HERE, "build")

SOURCES = [
    "pf_runtime.cpp",
    "pf_gemm.hip",
    "pf_attention.hip",
    "pf_norm.hip",
    "pf_elementwise.hip",
    "pf_softmax_loss.hip",
    "pf_batch.hip",
    "pf_mfma_rate.hip",
]

# the direct-to-LDS MFMA kernel: one object per (operand dtype id, tile id), all from one source
# (ids as in csrc/pf_gemm_common.h: dtypes PF_F16 = 1, PF_BF16 = 2; tiles PF_XT_* = 1..9)
GEMM_X_SOURCE = "pf_gemm_x_inst.hip"
GEMM_X_PAIRS = [(dt, xt) for xt in (1, 2, 3, 4, 5, 6, 7, 8, 9) for dt in (1, 2)]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

COMMON_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    "-Wno-unknown-attributes",
    "-Wno-pass-failed",
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _compile_one(job):
    src, defines, stem = job
    obj = os.path.join(OBJ_DIR, stem + ".o")
    cmd = [HIPCC, "-x", "hip"] + COMMON_FLAGS + defines + ["-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the packed-fp32 feature and says so once per pass
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, " ".join(cmd), err))
    return obj, err


def build(verbose=True, jobs=None):
    """Compile all sources and link the shared library. Always recompiles."""
    if not os.path.exists(HIPCC):
        raise RuntimeError("hipcc not found at %s (set HIPCC)" % HIPCC)
    os.makedirs(OBJ_DIR, exist_ok=True)
    work = [(GEMM_X_SOURCE, ["-DPF_X_DT=%d" % dt, "-DPF_X_TILE=%d" % xt], "pf_gemm_x_%d_%d" % (dt, xt))
            for dt, xt in GEMM_X_PAIRS]   # the long ones first
    work += [(src, [], os.path.splitext(src)[0]) for src in SOURCES]
    jobs = jobs or min(len(work), max(1, os.cpu_count() or 2))
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(_compile_one, work))
    objs = [o for o, _ in results]
    if verbose:
        for (_, warn), job in zip(results, work):
            if warn.strip():
                print("[pfeife_amd.hip.build] %s:\n%s" % (job[2], warn), file=sys.stderr)
    tmp = LIB_PATH + ".tmp"
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp] + objs
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (" ".join(cmd), res.stderr))
    os.replace(tmp, LIB_PATH)
    if verbose:
        print("[pfeife_amd.hip.build] built %s" % LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build()
