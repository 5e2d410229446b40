"""Host-side behaviour of bench.py that needs no GPU: the one-GPU rule, and the HBM-traffic record (written from two
rocprofv3 counter files, read back only while the measured kernels' sources hash the same)."""
import csv
import json
import os
import subprocess
import sys

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2
    assert "ONE GPU" in r.stderr and r.stdout.strip() == ""


def _counter_csv(path, counter, rows):
    with open(path, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=["Kernel_Name", "Counter_Name", "Counter_Value"])
        w.writeheader()
        for name, value in rows:
            w.writerow({"Kernel_Name": name, "Counter_Name": counter, "Counter_Value": value})


def test_traffic_record_scales_by_the_copy_and_is_dropped_when_the_sources_change(tmp_path, monkeypatch):
    kib = 256 << 10                                   # the calibration copy moves 256 MiB = 262144 KiB each way
    kernels = ["void mhffn::mhffn_fwd_kernel<128>(mhffn::FwdArgs)", "void mhffn::mhffn_bwd_dqdr_kernel<128>(mhffn::DqArgs)",
               "void mhffn::mhffn_bwd_dkdudv_kernel<128, false>(mhffn::DwArgs)"]
    # FETCH_SIZE under-reads by 2x on this counter set-up (the copy shows half its bytes); small copies must be ignored
    fetch = [("__amd_rocclr_copyBuffer", kib / 2)] * 4 + [("__amd_rocclr_copyBuffer", 10.0)] * 3 + \
            [(kernels[0], 1000.0), (kernels[0], 3000.0), (kernels[1], 500.0), (kernels[2], 250.0)]
    write = [("__amd_rocclr_copyBuffer", kib)] * 4 + [(kernels[0], 100.0), (kernels[1], 200.0), (kernels[2], 300.0)]
    fpath, wpath, out = tmp_path / "f.csv", tmp_path / "w.csv", tmp_path / "rec.json"
    _counter_csv(fpath, "FETCH_SIZE", fetch)
    _counter_csv(wpath, "WRITE_SIZE", write)
    bench.write_traffic_record("c2", str(fpath), str(wpath), str(out))
    rec = json.load(open(out))
    assert abs(rec["scale"]["FETCH_SIZE"] - 2.0) < 1e-9 and abs(rec["scale"]["WRITE_SIZE"] - 1.0) < 1e-9
    assert "bwd_reduce" not in rec["kernels"]          # no reduce launch in the files: one token slice
    k = rec["kernels"]["fwd_main"]
    assert k["launches"] == 2
    assert abs(k["fetch_bytes"] - 2000.0 * 1024 * 2.0) < 1e-6 and abs(k["write_bytes"] - 100.0 * 1024) < 1e-6
    assert abs(k["hbm_bytes"] - (k["fetch_bytes"] + k["write_bytes"])) < 1e-6
    assert rec["kernel_source_sha256"] == bench.kernel_source_hash()

    monkeypatch.setattr(bench, "traffic_record_path", lambda workload: str(out))
    got, note = bench.recorded_traffic("c2", "bwd_dkdudv")
    assert abs(got - (250.0 * 1024 * 2.0 + 300.0 * 1024)) < 1e-6 and "rocprofv3" in note
    monkeypatch.setattr(bench, "kernel_source_hash", lambda: "0" * 64)
    got, note = bench.recorded_traffic("c2", "bwd_dkdudv")
    assert got is None and "other kernel sources" in note


def test_the_committed_traffic_record_describes_the_committed_kernels():
    """profiles/c2_hbm_traffic.json must have been measured on the kernel sources in this tree (else bench.py reports
    traffic null): re-measure after every change to the three source files it hashes."""
    rec = json.load(open(os.path.join(ROOT, "profiles", "c2_hbm_traffic.json")))
    assert rec["kernel_source_sha256"] == bench.kernel_source_hash()
    assert set(rec["kernels"]) >= {"fwd_main", "bwd_dqdr", "bwd_dkdudv"}
