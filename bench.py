#!/usr/bin/env python3
"""Benchmark of the fused multi-head FFN hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|c1|c3|c4|c2_prologue|c3_prologue] [--no-cpu]

One "step" = one forward + one backward of the fused operator (through the C ABI, on torch's current stream) over
one synthetic batch already resident in HBM.  Prints ONE JSON line.  Credited FLOPs: F1 = 2*T*H*E*d_e*d_h per
GEMM; forward 3*F1, backward 8*F1 (recompute M,N + dA + 2 dQ + dK + dU + dV), fwd+bwd 11*F1 -- recomputation beyond
that (the two-kernel backward runs 11*F1 on the hardware, 14*F1 with the forward) is not credited.

Workload c4 is different in kind: one forward + backward of a whole random-init decoder (20 blocks of causal attention +
the MH-FFN block of workload c3's shape, vocabulary 50,304) on batch 2 x 4096 random token ids; it reports tokens/s and
peak memory only.

Workloads c2_prologue / c3_prologue time the block's head prologue (per-head RMSNorm + expert gate, forward and backward,
mhffn_gate_fwd / mhffn_gate_bwd) on the [B,S,H,d_h] heads of workloads c2 / c3.  These kernels are bound by HBM traffic:
the value is algorithmic bytes per second, forward 2|Q| + |R| (read x, write Q and R), backward 3|Q| + |R| (read x, dQ
and dR, write dx), |Q| = 2 T H d_h, |R| = 4 T H E; the router and norm weights and their gradients are a few KB per head.
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, published
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E, published

WORKLOADS = {
    # name: (B, S, hidden, H, d_h, E, d_e, passes)
    "c1": dict(B=8, S=2048, H=8, d_h=96, E=8, d_e=256, passes="fwd", label="128M layer fwd, bf16, 16384 tokens"),
    "c2": dict(B=8, S=2048, H=8, d_h=128, E=11, d_e=352, passes="fwd+bwd",
               label="370M layer fwd+bwd, bf16, B8xS2048=16384 tokens, H8 d_h128 E11 d_e352"),
    "c3": dict(B=4, S=8192, H=16, d_h=128, E=22, d_e=352, passes="fwd+bwd", label="1.3B layer fwd+bwd, bf16, 32768 tokens"),
    "c4": dict(B=2, S=4096, H=16, d_h=128, E=22, d_e=352, layers=20, vocab=50304, attn_heads=16, passes="model",
               label="1.3B decoder (20 blocks: causal MHA + MH-FFN H16 d_h128 E22 d_e352, RMSNorm, vocab 50304), "
                     "one bf16 forward+backward, B2xS4096 random token ids"),
    "c2_prologue": dict(B=8, S=2048, H=8, d_h=128, E=11, passes="prologue",
                        label="head prologue (per-head RMSNorm + expert gate) fwd+bwd on the 370M layer's heads, bf16, "
                              "B8xS2048 tokens, H8 d_h128 E11"),
    "c3_prologue": dict(B=4, S=8192, H=16, d_h=128, E=22, passes="prologue",
                        label="head prologue (per-head RMSNorm + expert gate) fwd+bwd on the 1.3B layer's heads, bf16, "
                              "B4xS8192 tokens, H16 d_h128 E22"),
}


def make_inputs(w, device, seed=0):
    """Synthetic inputs with the benchmark's distributions: Q ~ N(0,1) (X W_q with W_q ~ N(0,1/hid)),
    K,U,V ~ N(0, d_h^-1/2), gate logits X W_r with W_r ~ N(0, 0.02) -> sigmoid -> normalised over E, dO ~ N(0,1)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    B, S, H, dh, E, de = w["B"], w["S"], w["H"], w["d_h"], w["E"], w["d_e"]
    hid = H * dh
    Q = torch.randn(B, H, S, dh, generator=g).to(torch.bfloat16)
    K, U, V = ((torch.randn(H, E, de, dh, generator=g) * dh ** -0.5).to(torch.bfloat16) for _ in range(3))
    logits = torch.randn(B, H, S, E, generator=g) * (0.02 * hid ** 0.5)   # std of X @ W_r for X ~ N(0,1)
    R = torch.sigmoid(logits)
    R = (R / R.sum(-1, keepdim=True)).float()
    dO = torch.randn(B, H, S, dh, generator=g).to(torch.bfloat16)
    return [t.to(device) for t in (Q, K, U, V, R, dO)]


def f1(w):
    return 2.0 * w["B"] * w["S"] * w["H"] * w["E"] * w["d_e"] * w["d_h"]


def time_events(fn, n, warm=10):
    for _ in range(warm):
        fn()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(n):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / n


def kernel_timings(w, ins, n=50, sample_state=True):
    """Average duration of each kernel, bracketed by events on the launch stream (torch's current stream)."""
    from flashmhf_amd import _capi
    Q, K, U, V, R, dO = ins
    L = _capi.lib()
    dims = _capi.Dims(w["B"], w["H"], w["H"], w["S"], w["d_h"], w["E"], w["d_e"])
    O, dQ = torch.empty_like(Q), torch.empty_like(Q)
    dK, dU, dV = (torch.empty_like(K) for _ in range(3))
    dR = torch.empty_like(R)
    wsf = torch.empty(max(16, L.mhffn_fwd_workspace_bytes(dims, 0)), dtype=torch.uint8, device=Q.device)
    ws_bytes = L.mhffn_bwd_workspace_bytes(dims, 0)          # 0 where dK/dU/dV run as one token slice (no reduce pass)
    wsb = torch.empty(max(16, ws_bytes), dtype=torch.uint8, device=Q.device)
    st = torch.cuda.current_stream().cuda_stream

    def fwd(ph):
        rc = L.mhffn_fwd_phases(Q.data_ptr(), K.data_ptr(), U.data_ptr(), V.data_ptr(), R.data_ptr(), O.data_ptr(),
                                wsf.data_ptr(), wsf.numel(), dims, 0, st, ph)
        assert rc == 0, rc

    def bwd(ph):
        rc = L.mhffn_bwd_phases(Q.data_ptr(), K.data_ptr(), U.data_ptr(), V.data_ptr(), R.data_ptr(), dO.data_ptr(),
                                dQ.data_ptr(), dK.data_ptr(), dU.data_ptr(), dV.data_ptr(), dR.data_ptr(), 0,
                                wsb.data_ptr(), wsb.numel(), dims, 0, st, ph)
        assert rc == 0, rc

    fwd(_capi.FWD_ALL)
    runs = {"fwd_main": lambda: fwd(_capi.FWD_MAIN)}
    if "bwd" in w["passes"]:
        bwd(_capi.BWD_ALL)
        runs.update(bwd_dqdr=lambda: bwd(_capi.BWD_DQDR), bwd_dkdudv=lambda: bwd(_capi.BWD_DKDUDV))
        if ws_bytes:
            runs.update(bwd_reduce=lambda: bwd(_capi.BWD_REDUCE))
    out = {k: time_events(f, n) for k, f in runs.items()}
    state = {k: device_state_under(f) for k, f in runs.items() if k != "bwd_reduce"} if sample_state else {}
    return out, state


def device_sysfs_dir():
    """sysfs directory of the GPU torch runs on (cuda:0), found through its PCI address; with that unknown, the only
    card of the machine; None when several cards are visible and none can be matched."""
    import glob
    try:
        pr = torch.cuda.get_device_properties(0)
        d = f"/sys/bus/pci/devices/{pr.pci_domain_id:04x}:{pr.pci_bus_id:02x}:{pr.pci_device_id:02x}.0"
        if os.path.exists(os.path.join(d, "pp_dpm_sclk")):
            return d
    except (AttributeError, RuntimeError):
        pass
    cards = sorted(os.path.dirname(f) for f in glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
    return cards[0] if len(cards) == 1 else None


def settle_clock(fn, ms):
    """Runs `fn` back to back for at least `ms` milliseconds (untimed) and returns the time spent: the shader clock and
    the power controller need some tens of milliseconds of the workload itself before they stop moving."""
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(4):
            fn()
        torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3


def device_state_under(fn, seconds=0.5):
    """Shader clock (MHz) and package power (W) as the driver reports them (sysfs pp_dpm_sclk, hwmon power1_input)
    while `fn` is launched back to back for `seconds`: median of the samples taken after the first 100 ms.  The clock a
    kernel is given depends on the kernel: under matrix-heavy load the package sits at its power limit and the clock
    settles well below the 2.4 GHz the nominal peak is quoted at.  Returns None where the files cannot be read."""
    import threading
    card = device_sysfs_dir()
    if card is None:
        return None
    import glob
    sclk = glob.glob(os.path.join(card, "pp_dpm_sclk"))
    pwr = glob.glob(os.path.join(card, "hwmon", "hwmon*", "power1_input"))
    cap = glob.glob(os.path.join(card, "hwmon", "hwmon*", "power1_cap"))
    if not sclk:
        return None
    samples, stop = [], threading.Event()

    def read_mhz():
        for line in open(sclk[0]):
            if line.rstrip().endswith("*"):
                return float(line.split(":")[1].strip().split("M")[0])
        return None

    def sampler():
        t0 = time.perf_counter()
        while not stop.is_set():
            try:
                mhz = read_mhz()
                w = float(open(pwr[0]).read()) / 1e6 if pwr else None
                if time.perf_counter() - t0 > 0.1:
                    samples.append((mhz, w))
            except (OSError, ValueError, IndexError):
                pass
            time.sleep(0.004)

    th = threading.Thread(target=sampler, daemon=True)
    th.start()
    t_end = time.perf_counter() + seconds
    while time.perf_counter() < t_end:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
    stop.set()
    th.join()
    med = lambda xs: sorted(xs)[len(xs) // 2] if xs else None
    out = {"sclk_mhz": med([m for m, _ in samples if m]), "power_w": med([w for _, w in samples if w]),
           "samples": len(samples)}
    try:
        out["power_cap_w"] = float(open(cap[0]).read()) / 1e6 if cap else None
    except (OSError, ValueError):
        out["power_cap_w"] = None
    return out


def measured_mfma_peak_tflops(dev, random_data=False):
    """Rate of a register-resident v_mfma_f32_32x32x16_bf16 loop on every SIMD (mhffn_probe_mfma_loop), ~5 ms per launch.
    random_data: operand values in which every bit varies (as in real activations and weights) instead of small, smoothly
    varying ones; the package grants a lower clock for them."""
    import ctypes
    from flashmhf_amd import build as b
    L = ctypes.CDLL(b.PROBE_LIB)
    L.mhffn_probe_mfma_loop.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                        ctypes.POINTER(ctypes.c_double)]
    sink = torch.zeros(4, device=dev)
    flops = ctypes.c_double(0.0)
    blocks = torch.cuda.get_device_properties(dev).multi_processor_count
    st = torch.cuda.current_stream().cuda_stream

    def run():
        rc = L.mhffn_probe_mfma_loop(sink.data_ptr(), blocks, 10000, int(random_data), st, ctypes.byref(flops))
        assert rc == 0, rc

    ms = time_events(run, 5, warm=3)
    return flops.value / (ms * 1e-3) / 1e12, device_state_under(run, seconds=0.4)


# Credited GEMMs per kernel (in units of F1): the forward's three; the dQ/dR kernel's recomputed M, N, dA and the two
# dQ products; the dK/dU/dV kernel's three output products (its own recomputation of M, N, dA is not credited).
CREDIT = {"fwd_main": 3, "bwd_dqdr": 5, "bwd_dkdudv": 3}
HARDWARE = {"fwd_main": 3, "bwd_dqdr": 5, "bwd_dkdudv": 6}

# HBM bytes per launch cannot be read from inside this process: they come from two rocprofv3 --pmc runs of this very
# script (FETCH_SIZE, then WRITE_SIZE, with --calibrate-copy), which `--traffic-from` turns into a small JSON record
# under profiles/ together with a hash of the kernel sources.  A run whose kernel sources hash differently reports
# traffic null: the record no longer describes the kernels being timed.
TRAFFIC_KERNELS = {"fwd_main": "mhffn_fwd_kernel", "bwd_dqdr": "mhffn_bwd_dqdr_kernel",
                   "bwd_dkdudv": "mhffn_bwd_dkdudv_kernel", "bwd_reduce": "reduce_partials_kernel"}
TRAFFIC_SOURCES = ("mhffn_bwd.hip", "mhffn_common.hpp", "mhffn_fwd.hip")
COPY_KERNEL, COPY_BYTES = "__amd_rocclr_copyBuffer", 256 << 20


def traffic_record_path(workload):
    return os.path.join(ROOT, "profiles", f"{workload}_hbm_traffic.json")


def kernel_source_hash():
    import hashlib
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "flashmhf_amd", "csrc")
    for name in TRAFFIC_SOURCES:                     # the files the four measured kernels are compiled from
        h.update(name.encode())
        h.update(open(os.path.join(csrc, name), "rb").read())
    return h.hexdigest()


def write_traffic_record(workload, fetch_csv, write_csv, out_path):
    """rocprofv3 counter CSVs (one FETCH_SIZE run, one WRITE_SIZE run of `bench.py --calibrate-copy`) -> JSON record.
    Counter values are KiB per dispatch; each counter is scaled by what it reads for the 256 MiB device copy."""
    import csv

    def averages(path, counter):
        acc = {}
        with open(path, newline="") as f:
            for r in csv.DictReader(f):
                if r["Counter_Name"] == counter:
                    acc.setdefault(r["Kernel_Name"], []).append(float(r["Counter_Value"]))
        return {k: (sum(v) / len(v), len(v)) for k, v in acc.items()}

    def pick(avgs, needle):
        hits = [(v, n) for k, (v, n) in avgs.items() if needle in k]
        if not hits:
            raise SystemExit(f"no dispatch of {needle} in the counter file")
        return max(hits, key=lambda x: x[1])

    def copy_reading(path, counter):
        # the runtime's copy kernel also moves the small input tensors: the 256 MiB calibration copies are its largest
        # dispatches (four of them, equal to within counter noise)
        vals = []
        with open(path, newline="") as f:
            for r in csv.DictReader(f):
                if r["Counter_Name"] == counter and COPY_KERNEL in r["Kernel_Name"]:
                    vals.append(float(r["Counter_Value"]))
        big = [v for v in vals if v >= 0.9 * max(vals)] if vals else []
        if len(big) < 2:
            raise SystemExit("the calibration copies are missing: profile bench.py with --calibrate-copy")
        return sum(big) / len(big)

    fetch, write = averages(fetch_csv, "FETCH_SIZE"), averages(write_csv, "WRITE_SIZE")
    f_scale = (COPY_BYTES / 1024.0) / copy_reading(fetch_csv, "FETCH_SIZE")
    w_scale = (COPY_BYTES / 1024.0) / copy_reading(write_csv, "WRITE_SIZE")
    rec = {"workload": workload, "kernel_source_sha256": kernel_source_hash(),
           "command": "rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE --output-format csv -d <dir> -o p -- python3 bench.py "
                      f"--workload {workload} --no-cpu --no-others --steps 2 --warmup 1 --calibrate-copy ; python3 bench.py --workload "
                      f"{workload} --traffic-from <fetch csv> <write csv>",
           "scale": {"FETCH_SIZE": f_scale, "WRITE_SIZE": w_scale,
                     "reference": "256 MiB device copy (__amd_rocclr_copyBuffer) reads and writes 262144 KiB per launch"},
           "kernels": {}}
    for key, needle in TRAFFIC_KERNELS.items():
        if key == "bwd_reduce" and not any(needle in k for k in fetch):
            continue                                   # one token slice: dK/dU/dV are written by the kernel itself
        (fk, n), (wk, _) = pick(fetch, needle), pick(write, needle)
        rec["kernels"][key] = {"launches": n, "fetch_bytes": fk * 1024 * f_scale, "write_bytes": wk * 1024 * w_scale,
                               "hbm_bytes": fk * 1024 * f_scale + wk * 1024 * w_scale}
    with open(out_path, "w") as f:
        json.dump(rec, f, indent=1)
        f.write("\n")
    print(json.dumps(rec))


def recorded_traffic(workload, kernel):
    """(bytes per launch or None, note) for the dominant kernel from the committed counter record."""
    path = traffic_record_path(workload)
    if not os.path.exists(path):
        return None, "no counter record for this workload under profiles/"
    rec = json.load(open(path))
    if rec.get("kernel_source_sha256") != kernel_source_hash():
        return None, (f"profiles/{os.path.basename(path)} was measured on other kernel sources "
                      f"({rec.get('kernel_source_sha256', '?')[:12]}); rerun the two rocprofv3 --pmc passes")
    k = rec["kernels"].get(kernel)
    if not k:
        return None, f"kernel {kernel} not in profiles/{os.path.basename(path)}"
    return k["hbm_bytes"], f"profiles/{os.path.basename(path)} (rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE, scaled by a 256 MiB copy)"


def cpu_baseline(w, budget_s=25.0):
    """The CPU oracle (eager expert loop + torch.autograd, fp32) on a bounded sample of the same layer shape."""
    from oracle import mhffn_oracle as orc
    sample = dict(w, B=1, S=min(w["S"], 1024))
    g = torch.Generator().manual_seed(0)
    B, S, H, dh, E, de = (sample[k] for k in ("B", "S", "H", "d_h", "E", "d_e"))
    Q = torch.randn(B, H, S, dh, generator=g)
    K, U, V = (torch.randn(H, E, de, dh, generator=g) * dh ** -0.5 for _ in range(3))
    R = torch.softmax(torch.randn(B, H, S, E, generator=g), -1)
    dO = torch.randn(B, H, S, dh, generator=g)
    cores = torch.get_num_threads()
    bwd = "bwd" in w["passes"]

    def run():
        if bwd:
            orc.mhffn_autograd(Q, K, U, V, R, dO, compute_dtype=torch.float32)
        else:
            orc.mhffn_forward(Q, K, U, V, R, compute_dtype=torch.float32)

    run()
    times, t_start = [], time.perf_counter()
    while len(times) < 5 and (time.perf_counter() - t_start) < budget_s:
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    flops = (11 if bwd else 3) * f1(sample)
    return {"value": flops / med / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"oracle eager loop + autograd, fp32, B1xS{S} tokens of the same layer shape, median of {len(times)} runs, "
                      f"{med * 1e3:.1f} ms/step, tokens/s {B * S / med:.0f}"}


def cpu_baseline_c0():
    """The reference's CPU-runnable case: one 128M-config MH-FFN layer forward in fp32 through the layer wrapper
    (Q = X W_q split into heads, R = sigmoid(X W_r) normalised over E, eager expert loop, W_o;
    models/flashmhf/modeling_mhffnmoe.py:352-431) on X [2,128,768], H8 d_h96 E8 d_e256, seed 0;
    all host threads, 3 warm-ups, 10 timed runs, median and min."""
    import platform
    from oracle import mhffn_oracle as orc
    B, S, hid, H, E, de = 2, 128, 768, 8, 8, 256
    dh = hid // H
    g = torch.Generator().manual_seed(0)
    X = torch.randn(B, S, hid, generator=g)
    Wq, Wo = (torch.randn(hid, hid, generator=g) * hid ** -0.5 for _ in range(2))
    Wr = torch.randn(hid, H * E, generator=g) * 0.02
    K, U, V = (torch.randn(H, E, de, dh, generator=g) * dh ** -0.5 for _ in range(3))
    run = lambda: orc.mhffn_layer_forward(X, Wq, Wr, K, U, V, Wo, num_heads=H, compute_dtype=torch.float32)
    with torch.no_grad():
        for _ in range(3):
            run()
        times = []
        for _ in range(10):
            t0 = time.perf_counter()
            run()
            times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    flops = 3 * 2.0 * B * S * H * E * de * dh        # the fused path's three GEMMs; the two projections add 2*2*T*hid^2
    model = platform.processor() or ""
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return {"value": flops / med / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "median_ms": med * 1e3, "min_ms": times[0] * 1e3, "tokens_per_s": B * S / med, "cpu_model": model,
            "host_cpus": os.cpu_count(),
            "sample": "oracle layer wrapper forward (Q = X W_q, sigmoid gate from X W_r, eager expert loop, W_o), fp32, "
                      "B2xS128 hid 768 H8 d_h96 E8 d_e256, 3 warm-ups + 10 runs"}


def swiglu_peak_bytes(tokens, hidden, inner, device):
    """Peak HBM beyond inputs of a SwiGLU FFN (gate/up/down nn.Linear, bf16) fwd+bwd on the same tokens: the memory
    comparison of workload c3 (inner size from the reference's configs/baseline/configure10-TriDao-1.3B-bf16-pile.json:11)."""
    import torch.nn.functional as F
    x = torch.randn(tokens, hidden, device=device, dtype=torch.bfloat16, requires_grad=True)
    gate, up = (torch.nn.Linear(hidden, inner, bias=False, device=device, dtype=torch.bfloat16) for _ in range(2))
    down = torch.nn.Linear(inner, hidden, bias=False, device=device, dtype=torch.bfloat16)
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    y = down(F.silu(gate(x)) * up(x))
    y.backward(torch.ones_like(y))
    torch.cuda.synchronize()
    return int(torch.cuda.max_memory_allocated() - base)


def bench_model(w, args, dev):
    """Workload c4: one training step (forward + backward) of the whole decoder; tokens/s and peak memory."""
    from flashmhf_amd import MHFFNDecoder
    torch.manual_seed(0)
    hid = w["H"] * w["d_h"]
    with torch.device(dev):
        model = MHFFNDecoder(w["vocab"], hid, w["layers"], w["attn_heads"], w["H"], w["E"], w["d_e"],
                             apply_rmsnorm=True).to(torch.bfloat16)
    n_params = sum(p.numel() for p in model.parameters())
    ids = torch.randint(0, w["vocab"], (w["B"], w["S"]), device=dev, generator=torch.Generator(dev).manual_seed(0))

    def step():
        model.zero_grad(set_to_none=True)
        loss = model(ids, labels=ids)
        loss.backward()
        return loss

    for _ in range(args.warmup):
        loss = step()
    torch.cuda.synchronize()
    base_mem = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    tokens = w["B"] * w["S"]
    ffn_flops = w["layers"] * 11 * f1(w)
    out = {
        "metric": "1.3B decoder forward+backward tokens/s + peak memory, 1 GPU", "value": tokens / (ms * 1e-3),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"c4: {w['label']}", "parameters": n_params},
        "loss": float(loss.detach()),
        "peak_memory_bytes": {"max_allocated": int(torch.cuda.max_memory_allocated()),
                              "parameters_and_grads_before_step": int(base_mem)},
        "fused_ffn_credited_tflops_if_it_were_the_whole_step": ffn_flops / (ms * 1e-3) / 1e12,
        "roofline": None, "cpu_baseline": None,
    }
    del model
    torch.cuda.empty_cache()
    return out


def bench_prologue(w, args, dev):
    """Head prologue kernels through the C ABI on preallocated buffers: one step = forward + backward."""
    from flashmhf_amd import _capi
    B, S, H, dh, E = (w[k] for k in ("B", "S", "H", "d_h", "E"))
    g = torch.Generator().manual_seed(0)
    x = torch.randn(B, S, H, dh, generator=g).bfloat16().to(dev)
    wn = (torch.rand(H, dh, generator=g) + 0.5).to(dev)
    wr = (torch.randn(H, dh, E, generator=g) * 0.02 * (H * dh) ** 0.5 / dh ** 0.5).to(dev)
    dQ = torch.randn(B, S, H, dh, generator=g).bfloat16().to(dev)
    dR = torch.randn(B, H, S, E, generator=g).to(dev)
    Qn, dX = torch.empty_like(x), torch.empty_like(x)
    R = torch.empty(B, H, S, E, device=dev)
    dwn, dwr = torch.zeros_like(wn), torch.zeros_like(wr)
    L = _capi.lib()
    dims = _capi.Dims(B, H, H, S, dh, E, 32)
    st = torch.cuda.current_stream().cuda_stream

    def fwd():
        rc = L.mhffn_gate_fwd(x.data_ptr(), wn.data_ptr(), 1e-6, wr.data_ptr(), Qn.data_ptr(), R.data_ptr(), dims, st)
        assert rc == 0, rc

    def bwd():
        rc = L.mhffn_gate_bwd(x.data_ptr(), wn.data_ptr(), 1e-6, wr.data_ptr(), dQ.data_ptr(), _capi.TOKENS_BSHD,
                              dR.data_ptr(), dX.data_ptr(), dwn.data_ptr(), dwr.data_ptr(), dims, st)
        assert rc == 0, rc

    def step():
        fwd()
        bwd()

    pre_warm_ms = settle_clock(step, args.pre_warm_ms)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    q_bytes, r_bytes = 2.0 * B * S * H * dh, 4.0 * B * S * H * E
    alg = {"gate_fwd": 2 * q_bytes + r_bytes, "gate_bwd": 3 * q_bytes + r_bytes}
    kt = {"gate_fwd": time_events(fwd, 50), "gate_bwd": time_events(bwd, 50)}
    dom = max(kt, key=kt.get)
    ach = alg[dom] / (kt[dom] * 1e-3) / 1e9
    out = {
        "metric": "MH-FFN head prologue fwd+bwd GB/s (algorithmic bytes), 1 GPU", "value": sum(alg.values()) / (ms * 1e-3) / 1e9,
        "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "pre_warm_ms": pre_warm_ms,
        "config": {"workload": f"{args.workload}: {w['label']}", "algorithmic_bytes_per_step": sum(alg.values())},
        "tokens_per_s": B * S / (ms * 1e-3),
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": ach, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": ach / PEAK_HBM_GBS, "traffic": None},
        "kernels": {k: {"ms": v, "algorithmic_gbs": alg[k] / (v * 1e-3) / 1e9} for k, v in kt.items()},
    }
    if not args.no_cpu:
        from oracle import mhffn_oracle as orc
        xs = x[:1, :1024].float().cpu().requires_grad_(True)
        wns, wrs = wn.cpu().requires_grad_(True), wr.cpu().requires_grad_(True)
        dQs, dRs = dQ[:1, :1024].float().cpu().transpose(1, 2), dR[:1, :, :1024].cpu()

        def run():
            q, r = orc.head_norm_gate(xs, wns, wrs)
            torch.autograd.grad([q, r], [xs, wns, wrs], [dQs, dRs])

        run()
        times = []
        for _ in range(5):
            t0 = time.perf_counter()
            run()
            times.append(time.perf_counter() - t0)
        med = sorted(times)[2]
        frac = 1024.0 / (B * S)
        out["cpu_baseline"] = {"value": sum(alg.values()) * frac / med / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
                               "kind": "port", "sample": f"oracle head_norm_gate + autograd, fp32, B1xS1024 tokens of the "
                                                         f"same heads, median of 5 runs, {med * 1e3:.1f} ms"}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50,
                    help="untimed steps first: the GPU clock needs some tens of milliseconds of load to settle")
    ap.add_argument("--pre-warm-ms", type=float, default=200.0,
                    help="before the counted warm-up steps, run the workload untimed for this long so that the timed steps "
                         "do not fall into the clock's start-up transient (reported as pre_warm_ms)")
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-others", action="store_true",
                    help="default workload only: skip the short runs of the other configurations (c1, c3, head prologue, "
                         "c4 decoder) that are appended to the JSON line as `other_workloads`")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy a few times (known-size reference for HBM traffic counters)")
    ap.add_argument("--traffic-from", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no GPU work: turn the counter_collection.csv files of two rocprofv3 --pmc runs of this script "
                         "(FETCH_SIZE, WRITE_SIZE; both with --calibrate-copy) into profiles/<workload>_hbm_traffic.json")
    args = ap.parse_args()
    if args.traffic_from:
        return write_traffic_record(args.workload, args.traffic_from[0], args.traffic_from[1], traffic_record_path(args.workload))
    if args.gpus != 1:
        print("bench.py: this build runs the fused MH-FFN on ONE GPU; --gpus must be 1 "
              "(heads shard with no exchange and tokens with one all-reduce of dK, dU, dV, but no multi-GPU path is built)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the fused operator has no CPU path", file=sys.stderr)
        sys.exit(1)

    from flashmhf_amd import mhffn_backward, mhffn_forward
    dev = torch.device("cuda:0")
    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_()
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)           # reads 256 MiB, writes 256 MiB per launch
        torch.cuda.synchronize()
        del src, dst
    out = run_workload(args.workload, args, dev)
    if args.workload == "c2" and not args.no_others:
        # the other configurations, short runs without the CPU legs, so that one default invocation records them all
        sub = argparse.Namespace(**{**vars(args), "no_cpu": True, "steps": 20, "warmup": 5})
        keep = ("value", "unit", "ms_per_step", "steps", "warmup", "pre_warm_ms", "config", "frac_of_mfma_peak", "tokens_per_s", "peak_hbm_bytes",
                "peak_memory_bytes", "swiglu_2048_5504_peak_hbm_bytes_beyond_inputs", "kernels", "roofline", "loss")
        out["other_workloads"] = {}
        for name in ("c1", "c3", "c2_prologue", "c3_prologue", "c4"):
            sub.workload = name
            sub.steps, sub.warmup = (5, 2) if name == "c4" else (20, 5)
            r = run_workload(name, sub, dev, light=True)
            out["other_workloads"][name] = {k: r[k] for k in keep if k in r}
    print(json.dumps(out))


def run_workload(name, args, dev, light=False):
    """One workload -> its result record.  light: no clock/power sampling, no matrix-loop probe, no autograd-operator timing."""
    from flashmhf_amd import mhffn_backward, mhffn_forward
    w = WORKLOADS[name]
    if w["passes"] == "model":
        return bench_model(w, args, dev)
    if w["passes"] == "prologue":
        return bench_prologue(w, args, dev)
    ins = make_inputs(w, dev)
    Q, K, U, V, R, dO = ins
    bwd = "bwd" in w["passes"]

    def step():
        O = mhffn_forward(Q, K, U, V, R)
        if bwd:
            return O, mhffn_backward(Q, K, U, V, R, dO, grad_w_dtype=torch.bfloat16)
        return O

    pre_warm_ms = settle_clock(step, args.pre_warm_ms)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    base_mem = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    peak_extra = torch.cuda.max_memory_allocated() - base_mem
    ms = dt / args.steps * 1e3
    flops = (11 if bwd else 3) * f1(w)
    tflops = flops / (ms * 1e-3) / 1e12
    tokens = w["B"] * w["S"]

    # per-step spread (one event pair per step) and the same step through the autograd operator
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(min(args.steps, 100))]
    for a, b in evs:
        a.record()
        step()
        b.record()
    torch.cuda.synchronize()
    per_step = sorted(a.elapsed_time(b) for a, b in evs)
    timing = {"median_ms": per_step[len(per_step) // 2], "min_ms": per_step[0]}
    if bwd and not light:
        from flashmhf_amd import FlashMLPMoE
        op = FlashMLPMoE()
        leaves = [t.detach().clone().requires_grad_(True) for t in (Q, K, U, V, R)]

        def autograd_step():
            for t in leaves:
                t.grad = None
            op(*leaves).backward(dO)

        timing["autograd_op_ms"] = time_events(autograd_step, min(args.steps, 100))

    kt, kstate = kernel_timings(w, ins, sample_state=not light)
    mfma_loop, probe_state = (None, None) if light else measured_mfma_peak_tflops(dev)
    mfma_loop_rnd, probe_state_rnd = (None, None) if light else measured_mfma_peak_tflops(dev, random_data=True)
    dom = max(CREDIT, key=lambda k: kt.get(k, 0.0))
    ach = CREDIT[dom] * f1(w) / (kt[dom] * 1e-3) / 1e12
    traffic, traffic_note = recorded_traffic(name, dom)
    roofline = {"bound": "mfma", "kernel": dom, "achieved": ach, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                "frac": ach / PEAK_BF16_TFLOPS, "traffic": traffic, "traffic_source": traffic_note,
                "hardware_tflops": HARDWARE[dom] * f1(w) / (kt[dom] * 1e-3) / 1e12}
    kernels = {k: {"ms": v, **({"credited_tflops": CREDIT[k] * f1(w) / (v * 1e-3) / 1e12,
                                "hardware_tflops": HARDWARE[k] * f1(w) / (v * 1e-3) / 1e12} if k in CREDIT else {}),
                   **({"under_load": kstate[k]} if kstate.get(k) else {})}
               for k, v in kt.items()}

    out = {
        "metric": "fused MH-FFN fwd+bwd TFLOP/s (% MFMA peak) + peak HBM, 370M layer, 1 GPU" if name == "c2"
                  else f"fused MH-FFN {w['passes']} TFLOP/s, workload {name}",
        "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic", "pre_warm_ms": pre_warm_ms,
        "config": {"workload": f"{name}: {w['label']}", "credited_flops_per_step": flops,
                   "flop_convention": "11*F1 fwd+bwd (3 fwd + 8 bwd), F1=2*T*H*E*d_e*d_h"},
        "frac_of_mfma_peak": tflops / PEAK_BF16_TFLOPS,
        "measured_mfma_loop_tflops": mfma_loop,
        "measured_mfma_loop_under_load": probe_state,
        "measured_mfma_loop_random_operands_tflops": mfma_loop_rnd,
        "measured_mfma_loop_random_operands_under_load": probe_state_rnd,
        "nominal_peak_clock_mhz": 2400,
        "frac_of_measured_mfma_loop": tflops / mfma_loop if mfma_loop else None,
        "tokens_per_s": tokens / (ms * 1e-3),
        "peak_hbm_bytes": {"beyond_inputs": int(peak_extra), "inputs": int(base_mem),
                           "forbidden_intermediate_bytes_one_tensor": tokens * w["H"] * w["E"] * w["d_e"] * 2},
        "roofline": roofline,
        "kernels": kernels,
        "timing": timing,
    }
    if name == "c3":
        out["swiglu_2048_5504_peak_hbm_bytes_beyond_inputs"] = swiglu_peak_bytes(tokens, 2048, 5504, dev)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(w)
        out["cpu_baseline_c0"] = cpu_baseline_c0()
    del ins, Q, K, U, V, R, dO
    torch.cuda.empty_cache()
    return out


if __name__ == "__main__":
    main()
