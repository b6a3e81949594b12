"""Compiles the HIP kernels into conef_amd/lib/libconef_hip.so (gfx950 only).

hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is installed.
The library is built in-tree; nothing is JIT-compiled at run time.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")     # the public C header, for the batch item struct
LIBDIR = os.path.join(HERE, "lib")
LIBPATH = os.path.join(LIBDIR, "libconef_hip.so")
# same sources with -DCONEF_TRACE: the two binned passes also write per-workgroup phase timestamps,
# read back with conef_trace_read (a measuring build; nothing in the package loads it)
TRACE_LIBPATH = os.path.join(LIBDIR, "libconef_hip_trace.so")

SOURCES = ["conef_sketch.hip", "conef_randblock.hip", "conef_randblock_batch.hip", "conef_psgd.hip", "conef_topk.hip",
           "conef_plan.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",          # every fused multiply-add in the kernels is an explicit fmaf
    "-munsafe-fp-atomics",        # hardware float atomics (LDS and L2) instead of CAS loops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; the ConEF HIP library cannot be built")


def build(verbose=False, trace=False):
    hipcc = _hipcc()
    os.makedirs(LIBDIR, exist_ok=True)
    objdir = os.path.join(LIBDIR, "obj_trace" if trace else "obj")
    flags = HIPCC_FLAGS + (["-DCONEF_TRACE"] if trace else [])
    libpath = TRACE_LIBPATH if trace else LIBPATH
    os.makedirs(objdir, exist_ok=True)
    sources = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc] + flags + ["-I", CSRC, "-I", INCLUDE, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s\n%s" % (src, res.stdout, res.stderr))
        if verbose and res.stderr.strip():
            print(res.stderr, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(6, len(sources))) as pool:
        objs = list(pool.map(compile_one, sources))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", libpath] + objs
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (res.stdout, res.stderr))
    return libpath


if __name__ == "__main__":
    print(build(verbose=True, trace="--trace" in sys.argv[1:]))
