"""The build's resource check (flashmhf_amd/build.py): the hand-scheduled kernels must compile without private (scratch)
memory, the one known exception is named, and a compiler whose remarks can no longer be parsed must not pass silently."""
import os

import pytest

from flashmhf_amd import build


def _usage(extra=None, drop=None, scratch=None):
    names = []
    for dh in (64, 96, 128):
        names += [f"_ZN5mhffn16mhffn_fwd_kernelILi{dh}EEEvNS_7FwdArgsE", f"_ZN5mhffn21mhffn_bwd_dqdr_kernelILi{dh}EEEvNS_6DqArgsE"]
        names += [f"_ZN5mhffn23mhffn_bwd_dkdudv_kernelILi{dh}ELb{t}EEEvNS_6DwArgsE" for t in (0, 1)]
        for nt in (1, 2):
            for norm in (0, 1):
                names += [f"_ZN5mhffn21mhffn_gate_{d}_kernelILi{dh}ELi{nt}ELb{norm}EEEvNS_8GateArgsE" for d in ("fwd", "bwd")]
    u = {n: {"ScratchSize": "0", "VGPRs": "100"} for n in names if not (drop and drop in n)}
    for k, v in (scratch or {}).items():
        hit = [n for n in u if k in n]
        assert hit, k
        for n in hit:
            u[n]["ScratchSize"] = str(v)
    u.update(extra or {})
    return u


def test_clean_usage_passes_and_unrelated_kernels_may_spill():
    build.check_no_scratch(_usage(extra={"_ZN5mhffn12_GLOBAL__N_117dkdudv_f32_kernelENS0_7F32ArgsE": {"ScratchSize": "64"}}))


def test_a_spill_in_a_hand_scheduled_kernel_fails_the_build():
    for frag in ("mhffn_fwd_kernelILi128E", "mhffn_bwd_dqdr_kernelILi96E", "mhffn_bwd_dkdudv_kernelILi64ELb1E",
                 "mhffn_gate_bwd_kernelILi128ELi1ELb1E", "mhffn_gate_fwd_kernelILi96ELi2ELb0E"):
        with pytest.raises(RuntimeError, match="scratch"):
            build.check_no_scratch(_usage(scratch={frag: 8}))


def test_the_named_exception_is_the_only_one():
    build.check_no_scratch(_usage(scratch={"mhffn_gate_bwd_kernelILi128ELi2ELb1E": 452}))
    with pytest.raises(RuntimeError, match="scratch"):
        build.check_no_scratch(_usage(scratch={"mhffn_gate_bwd_kernelILi128ELi2ELb0E": 452}))


def test_missing_remarks_fail_instead_of_passing_vacuously():
    with pytest.raises(RuntimeError, match="expected resource-usage remarks"):
        build.check_no_scratch({})
    with pytest.raises(RuntimeError, match="mhffn_bwd_dkdudv_kernel"):
        build.check_no_scratch(_usage(drop="mhffn_bwd_dkdudv_kernelILi96ELb1E"))


def test_remark_parser_reads_hipcc_output():
    text = ("x.hip:1:1: remark: Function Name: _ZN5mhffn16mhffn_fwd_kernelILi128EEEvNS_7FwdArgsE [-Rpass-analysis=kernel-resource-usage]\n"
            "x.hip:1:1: remark:     VGPRs: 239 [-Rpass-analysis=kernel-resource-usage]\n"
            "x.hip:1:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]\n"
            "x.hip:1:1: remark:     Occupancy [waves/SIMD]: 1 [-Rpass-analysis=kernel-resource-usage]\n")
    u = build.parse_resource_usage(text)
    assert u == {"_ZN5mhffn16mhffn_fwd_kernelILi128EEEvNS_7FwdArgsE": {"VGPRs": "239", "ScratchSize": "0", "Occupancy": "1"}}


def test_the_committed_resource_listing_is_clean():
    """flashmhf_amd/_lib/resource_usage.txt is what the last build wrote: it must satisfy the same check."""
    path = os.path.join(build.LIBDIR, "resource_usage.txt")
    if not os.path.exists(path):
        pytest.skip("library not built")
    usage = {}
    for line in open(path):
        name, *fields = line.split("  ")
        usage[name] = dict(f.strip().split("=", 1) for f in fields if "=" in f)
    build.check_no_scratch(usage)
