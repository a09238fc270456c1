"""Headline benchmark: butterfly_multiply forward + backward, batch 16384, n = 1024, fp32,
nblocks = 2, decreasing stride first, on one MI355X, through torch.ops.torch_butterfly.

    python bench.py [--steps K] [--warmup W] [--no-cpu-baseline]

Prints one JSON line.  ``value`` is algorithmic bytes (5 row-passes + twiddle traffic) per
second over the K timed forward+backward steps with operands resident in HBM.  ``roofline``
describes the dominant call, the backward pass, timed with device events on the launch
stream.  ``cpu_baseline`` is the single-threaded reference C++ (or, where that build is
absent, the repo's CPU restatement) timed on this host.
"""
import argparse
import json
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "butterfly_multiply fwd+bwd GB/s & % HBM peak, batch 16384 n=1024 fp32"
HBM_PEAK_GBS = 8000.0
BW_TRAFFIC_BYTES = 289.4e6

BATCH, NSTACKS, LOG_N, NBLOCKS, INCREASING = 16384, 1, 10, 2, False


def algorithmic_bytes():
    n = 1 << LOG_N
    row = NSTACKS * n * 4
    twiddle = NSTACKS * NBLOCKS * LOG_N * (n // 2) * 4 * 4
    fw = 2 * row * BATCH + twiddle                 # read input, write output, read twiddle
    bw = 3 * row * BATCH + 2 * twiddle             # read input + grad, write d_input; twiddle in, d_twiddle out
    return fw, bw


def cpu_baseline():
    """Reference csrc/cpu path (one thread) on the full workload, best of 3."""
    ref_so = os.path.join(ROOT, "oracle", "_ref", "_butterfly_ref.so")
    fw_b, bw_b = algorithmic_bytes()
    if os.path.isfile(ref_so):
        out = subprocess.check_output(
            [sys.executable, os.path.join(ROOT, "oracle", "ref_runner.py"), "time", str(BATCH), str(NSTACKS),
             str(LOG_N), str(NBLOCKS), str(int(INCREASING)), "0", "3"], text=True)
        r = json.loads(out.strip().splitlines()[-1])
        fw_s, bw_s, kind = r["fw_s"], r["bw_s"], "reference"
    else:
        import numpy as np
        from oracle import oracle
        rng = np.random.default_rng(0)
        n = 1 << LOG_N
        tw = (rng.standard_normal((NSTACKS, NBLOCKS, LOG_N, n // 2, 2, 2)) / np.sqrt(2)).astype(np.float32)
        x = rng.standard_normal((BATCH, NSTACKS, n)).astype(np.float32)
        g = rng.standard_normal((BATCH, NSTACKS, n)).astype(np.float32)
        fw_s = bw_s = float("inf")
        for _ in range(3):
            t0 = time.perf_counter(); oracle.butterfly_fw(tw, x, INCREASING)
            t1 = time.perf_counter(); oracle.butterfly_bw(tw, x, g, INCREASING)
            t2 = time.perf_counter()
            fw_s, bw_s = min(fw_s, t1 - t0), min(bw_s, t2 - t1)
        kind = "port"
    total = fw_s + bw_s
    return {"value": (fw_b + bw_b) / total / 1e9, "unit": "GB/s", "cores": 1, "kind": kind,
            "sample": f"full workload, batch {BATCH}, best of 3 (fw {fw_s * 1e3:.0f} ms, bw {bw_s * 1e3:.0f} ms)",
            "rows_per_s": BATCH / total}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run plain 64 MiB device copies (a kernel of known traffic, for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU; --gpus must be 1 (rows shard trivially, see DESIGN.md)")

    import torch
    import butterfly_amd  # noqa: F401
    ops = torch.ops.torch_butterfly
    assert torch.cuda.is_available(), "bench.py needs a HIP device"
    torch.manual_seed(0)
    n = 1 << LOG_N
    dev = torch.device("cuda:0")
    twiddle = (torch.randn(NSTACKS, NBLOCKS, LOG_N, n // 2, 2, 2) / 2 ** 0.5).to(dev)
    x = torch.randn(BATCH, NSTACKS, n).to(dev)
    grad = torch.randn(BATCH, NSTACKS, n).to(dev)

    def step():
        y = ops.butterfly_multiply_fw(twiddle, x, INCREASING, None)
        dtw, dx = ops.butterfly_multiply_bw(twiddle, x, grad, INCREASING)
        return y, dtw, dx

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    if args.calibrate_copy:
        dst = torch.empty_like(x)
        for _ in range(5):
            dst.copy_(x)
        torch.cuda.synchronize()
    fw_ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    bw_ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        fw_ev[i][0].record()
        ops.butterfly_multiply_fw(twiddle, x, INCREASING, None)
        fw_ev[i][1].record()
        bw_ev[i][0].record()
        ops.butterfly_multiply_bw(twiddle, x, grad, INCREASING)
        bw_ev[i][1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    fw_ms = sum(a.elapsed_time(b) for a, b in fw_ev) / args.steps
    bw_ms = sum(a.elapsed_time(b) for a, b in bw_ev) / args.steps
    ms_per_step = wall * 1e3 / args.steps
    fw_b, bw_b = algorithmic_bytes()
    value = (fw_b + bw_b) / (ms_per_step * 1e-3) / 1e9
    bw_gbs = bw_b / (bw_ms * 1e-3) / 1e9
    line = {
        "metric": METRIC, "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "cfg2: butterfly_multiply fw+bw, input (16384,1,1024) fp32 N(0,1), twiddle "
                               "(1,2,10,512,2,2) N(0,1/2), increasing_stride=False, grad N(0,1)"},
        "pct_hbm_peak": 100.0 * value / HBM_PEAK_GBS,
        "rows_per_s": BATCH / (ms_per_step * 1e-3),
        "fw_ms": fw_ms, "bw_ms": bw_ms,
        "fw_GBps": fw_b / (fw_ms * 1e-3) / 1e9,
        "roofline": {"bound": "hbm", "kernel": "butterfly_multiply_bw (main kernel + partial-sum reduce)",
                     "achieved": bw_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": bw_gbs / HBM_PEAK_GBS,
                     # HBM bytes per backward call (main kernel + reduce) from rocprofv3 FETCH_SIZE /
                     # WRITE_SIZE scaled by a 64 MiB copy; see profiles/butterfly_fw_bw_cfg2_hbm_traffic.md
                     "traffic": BW_TRAFFIC_BYTES},
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline()
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
