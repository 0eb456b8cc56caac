"""Compiles the HIP sources under featgraph_amd/csrc into featgraph_amd/lib/libfeatgraph_hip.so.

hipcc cross-compiles for gfx950 without a GPU present.  Run as
`python -m featgraph_amd.build`; tests, the smoke check and the benchmark load
the library that is already built and only build when none exists.
"""
import concurrent.futures
import os
import subprocess
import sys

_PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_PKG, "csrc")
LIB_DIR = os.path.join(_PKG, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libfeatgraph_hip.so")
SOURCES = ("api.hip", "spmm.hip", "spmm_multi.hip", "spmm_multi_general_mul.hip", "spmm_multi_general_add.hip",
           "spmm_multi_general_sub.hip", "spmm_multi_general_div.hip", "spmm_multi_general_copy_u.hip", "sddmm.hip", "sddmm_blocked.hip", "sddmm_sorted.hip", "noalloc.hip", "probe.hip", "general.hip", "softmax.hip", "attention.hip", "backward.hip")

# -ffp-contract=off: the SpMM kernels must round the product and the sum
# separately (fused multiply-adds are written explicitly where wanted).
# The target-feature pair switches packed-fp32 instructions off.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-command-line-argument",
]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _compile(src):
    obj = os.path.join(LIB_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    return src, obj, proc.returncode, proc.stdout


def build_hip(verbose=True):
    """Compile every HIP source and link the shared library.  Raises on failure."""
    os.makedirs(LIB_DIR, exist_ok=True)
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=len(SOURCES)) as pool:
        for src, obj, rc, log in pool.map(_compile, SOURCES):
            # the host pass does not know the GPU-only target feature; that warning is harmless
            log = "\n".join(l for l in log.splitlines() if "packed-fp32-ops" not in l)
            if verbose and log.strip():
                print(log, file=sys.stderr)
            if rc != 0:
                raise RuntimeError("hipcc failed on %s:\n%s" % (src, log))
            objs.append(obj)
    tmp = LIB_PATH + ".tmp"
    subprocess.check_call([_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs])
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_hip())
