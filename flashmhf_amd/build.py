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
SOURCES = ["mhffn_capi.hip", "mhffn_fwd.hip", "mhffn_bwd.hip", "mhffn_f32.hip", "mhffn_gate.hip"]
# benchmark-only object: a register-resident matrix-instruction loop bench.py times beside the kernels
PROBE_LIB = os.path.join(LIBDIR, "libmhffn_probe.so")
PROBE_SOURCE = "mhffn_probe.hip"
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

    usage = {}

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc, *FLAGS, "-Rpass-analysis=kernel-resource-usage", "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, stderr=subprocess.PIPE, text=True)
        other = [ln for ln in r.stderr.splitlines()
                 if "packed-fp32-ops" not in ln and "kernel-resource-usage" not in ln and (r.returncode or "warning" in ln or "error" in ln)]
        if other:
            print("\n".join(other), file=sys.stderr, flush=True)
        if r.returncode:
            raise subprocess.CalledProcessError(r.returncode, cmd)
        usage.update(parse_resource_usage(r.stderr))
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, SOURCES + [PROBE_SOURCE]))
    for out, members in ((LIB, objs[:-1]), (PROBE_LIB, objs[-1:])):
        cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out, *members]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    with open(os.path.join(LIBDIR, "resource_usage.txt"), "w") as f:     # registers, scratch, occupancy per kernel
        for name in sorted(usage):
            f.write(name + "  " + "  ".join(f"{k}={v}" for k, v in usage[name].items()) + "\n")
    check_no_scratch(usage)
    return LIB


def parse_resource_usage(stderr_text):
    """{kernel symbol: {field: value}} from hipcc's -Rpass-analysis=kernel-resource-usage remarks."""
    import re
    usage, cur = {}, None
    for line in stderr_text.splitlines():
        m = re.search(r"remark:\s+Function Name: (\S+)", line)
        if m:
            cur = usage.setdefault(m.group(1), {})
            continue
        m = re.search(r"remark:\s+([A-Za-z ]+?)(?: \[[^\]]*\])?: (\S+) \[-Rpass", line)
        if m and cur is not None:
            cur[m.group(1).strip()] = m.group(2)
    return usage


def check_no_scratch(usage):
    """The hand-scheduled kernels assume every value stays in registers: a spill would put VALU copies of matrix results
    into places the explicit wait states do not cover.  Fails the build if the compiler reports private (scratch)
    memory for one of them."""
    for name, u in usage.items():
        if ("mhffn_fwd_kernel" in name or "mhffn_bwd_" in name) and int(u.get("ScratchSize", "0")) != 0:
            raise RuntimeError(f"{name} uses {u['ScratchSize']} bytes of scratch per lane: a spill in a hand-scheduled kernel")


if __name__ == "__main__":
    print(build_lib(verbose="-q" not in sys.argv))
