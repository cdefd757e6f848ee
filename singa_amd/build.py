"""Builds the gfx950 shared library (``singa_amd/lib/libsinga_hip.so``) with hipcc.

Run as ``python -m singa_amd.build``.  The library is built in-tree; nothing is installed.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIBPATH = os.path.join(LIBDIR, "libsinga_hip.so")

SOURCES = ["runtime.hip", "eltwise.hip", "pool.hip", "batchnorm.hip", "igemm.hip", "wgrad3x3.hip", "conv16.hip",
    "wgrad_fewc.hip", "dgrad3x3.hip", "dgrad_fewc.hip", "half.hip", "tensor_fns.hip", "pointwise.hip", "fwd_fewc16.hip", "fwd_fewc.hip", "gemm16.hip"]

# Packed-FP32 VALU ops are disabled for every device code object of this library.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def build_library(verbose=True, jobs=4):
    """Compile every HIP source for gfx950 and link the shared library.  Always recompiles."""
    os.makedirs(LIBDIR, exist_ok=True)
    objdir = os.path.join(LIBDIR, "obj")
    os.makedirs(objdir, exist_ok=True)
    cc = hipcc()
    procs = []
    objs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = [cc] + HIPCC_FLAGS + ["-I", os.path.join(ROOT, "include"), "-I", CSRC, "-c",
                                    os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    cmd = [cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIBPATH] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIBPATH


def _drain(procs):
    while procs:
        src, p = procs.pop(0)
        out = p.communicate()[0].decode(errors="replace")
        # the host pass of hipcc does not know the device-only feature flag; that note is harmless
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if out.strip():
            print(out, flush=True)
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s" % src)


if __name__ == "__main__":
    build_library()
    print("built", LIBPATH)
    sys.exit(0)
