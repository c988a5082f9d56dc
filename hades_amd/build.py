"""Builds libhades_hip.so (the C-ABI library of HIP kernels for gfx950) in-tree with hipcc.

    python -m hades_amd.build          # compile every csrc/*.hip and link csrc/libhades_hip.so

hipcc cross-compiles for gfx950 without a GPU.  The library is loaded by hades_amd._lib.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB_NAME = "libhades_hip.so"
LIB_PATH = os.path.join(CSRC, LIB_NAME)

HIPCC_FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    # keep hipcc from forming packed-fp32 instructions out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
# Row-update arithmetic is compared bit-for-bit with a CPU restatement that rounds after every
# operation: forbid fused multiply-add contraction in device code.
NO_CONTRACT = ["-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt"]


def hipcc_path():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or put /opt/rocm/bin on PATH)")


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile_one(hipcc, src, verbose):
    obj = os.path.join(CSRC, src[:-4] + ".o")
    cmd = [hipcc] + HIPCC_FLAGS + NO_CONTRACT + ["-c", os.path.join(CSRC, src), "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the packed-fp32 target feature and says so: harmless
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s\n%s" % (src, res.stdout, res.stderr))
    if verbose and err.strip():
        print(err, flush=True)
    return obj


def build(verbose=True, jobs=None):
    """Compile every kernel source and link the shared library.  Always recompiles."""
    hipcc = hipcc_path()
    srcs = sources()
    jobs = jobs or min(len(srcs), int(os.environ.get("MAX_JOBS", "8")))
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile_one(hipcc, s, verbose), srcs))
    cmd = [hipcc, "-shared", "--offload-arch=gfx950", "-o", LIB_PATH] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (res.stdout, res.stderr))
    return LIB_PATH


if __name__ == "__main__":
    path = build(verbose="-q" not in sys.argv)
    print("built", path)
