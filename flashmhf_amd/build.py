"""Builds libmhffn_hip.so (the C-ABI library) in-tree with hipcc for gfx950.

    python -m flashmhf_amd.build

One code object, one architecture; no CUDA headers, no torch headers, links only libamdhip64.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "_lib")
LIB = os.path.join(LIBDIR, "libmhffn_hip.so")
SOURCES = ["mhffn_capi.hip", "mhffn_fwd.hip", "mhffn_bwd.hip", "mhffn_f32.hip", "mhffn_gate.hip", "mhffn_probe.hip"]
FLAGS = [
    "-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17",
    # packed fp32 VALU ops are kept out of the generated code on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def build_lib(verbose=False, jobs=4):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(LIBDIR, exist_ok=True)
    objdir = os.path.join(LIBDIR, "obj")
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        extra = os.environ.get("MHFFN_EXTRA_HIPCC_FLAGS", "").split()   # experiments only, e.g. -DSOME_TUNABLE=3
        cmd = [hipcc, *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    print(build_lib(verbose="-q" not in sys.argv))
