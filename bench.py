"""Benchmark of the butterfly multiply on one MI355X, through torch.ops.torch_butterfly.

    python bench.py [--steps K] [--warmup W] [--settle-ms T] [--config cfg2] [--no-cpu-baseline] [--calibrate-copy]

The default workload (cfg2) is the headline one: forward + backward, batch 16384, n = 1024,
fp32, nblocks = 2, decreasing stride first.  The other configurations of the baseline list
(cfg1, cfg3, cfg4, cfg5) can be selected with --config.  One JSON line is printed.

``value`` is algorithmic bytes (2 row passes forward, 3 backward, plus twiddle traffic) per
second over the K timed steps, operands resident in HBM.  Before the W warmup steps the same
step runs untimed for T milliseconds (default 250): the GPU needs a few tens of milliseconds
of sustained load to reach its steady clocks, and K steps of a 0.2 ms workload would
otherwise be timed entirely inside that ramp.  The K steps are then timed twice: once with
nothing between them (host clock around two device synchronisations: ``value``, ``ms_per_step``)
and once with a device event between consecutive calls on the launch stream (``fw_ms``,
``bw_ms``).  ``roofline`` describes the dominant call (the backward pass where there is one)
from those events, and the dominant kernel by itself (``kernel_name``, ``kernel_us``) from the
committed rocprofv3 kernel-trace summary of the same command.  ``cpu_baseline`` is the single-threaded reference C++ (or, for base-4 and where the
reference build is absent, the repo's CPU restatement) timed on this host on a bounded sample.
"""
import argparse
import json
import math
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

VALU_PEAK_TFLOPS = 157.3   # MI355X fp32 vector / matrix peak
HBM_PEAK_GBS = 8000.0
TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "hbm_traffic_all_configs.md")
KERNEL_SOURCES = os.path.join(ROOT, "butterfly_amd", "csrc")


def kernel_source_digest():
    """Digest of the library's sources: counter readings belong to the build they were taken on."""
    import hashlib
    h = hashlib.sha256()
    for name in sorted(os.listdir(KERNEL_SOURCES)):
        if name.endswith((".hpp", ".hip", ".cpp")):
            with open(os.path.join(KERNEL_SOURCES, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


def measured_traffic(config):
    """HBM bytes per launch set of the dominant call of `config`, from the rocprofv3 FETCH_SIZE /
    WRITE_SIZE table under profiles/ (a line `| config | digest | bytes | ...`), or None when
    there is no reading for this configuration or the sources have changed since it was taken."""
    try:
        with open(TRAFFIC_TABLE) as f:
            lines = f.read().splitlines()
    except OSError:
        return None
    digest = kernel_source_digest()
    for line in lines:
        cells = [c.strip().strip("`") for c in line.strip().strip("|").split("|")]
        if len(cells) >= 3 and cells[0] == config and cells[1] == digest:
            try:
                return float(cells[2])
            except ValueError:
                return None
    return None

KERNEL_TABLE = os.path.join(ROOT, "profiles", "kernel_trace_all_configs.md")


def measured_kernel(config):
    """(rocprof kernel name, average microseconds per launch, algorithmic bytes per launch) of the
    dominant kernel of `config`, from the `rocprofv3 --kernel-trace --stats` table under profiles/
    (a line `| config | digest | kernel | us | bytes |`), or None when there is no reading for this
    configuration or the sources have changed since it was taken."""
    try:
        with open(KERNEL_TABLE) as f:
            lines = f.read().splitlines()
    except OSError:
        return None
    digest = kernel_source_digest()
    for line in lines:
        cells = [c.strip().strip("`") for c in line.strip().strip("|").split("|")]
        if len(cells) >= 5 and cells[0] == config and cells[1] == digest:
            try:
                return cells[2], float(cells[3]), float(cells[4])
            except ValueError:
                return None
    return None


CONFIGS = {
    # name: batch, nstacks, log_n, nblocks, increasing_stride, complex, base4, backward, cpu sample batch
    "cfg1": dict(batch=2048, nstacks=1, log_n=10, nblocks=1, inc=True, cplx=False, base4=False, bw=False,
                 cpu_batch=2048,
                 metric="butterfly_multiply_fw GB/s, batch 2048 n=1024 fp32",
                 workload="cfg1: butterfly_multiply_fw, input (2048,1,1024) fp32 N(0,1), twiddle (1,1,10,512,2,2) "
                          "N(0,1/2), increasing_stride=True, forward only"),
    "cfg2": dict(batch=16384, nstacks=1, log_n=10, nblocks=2, inc=False, cplx=False, base4=False, bw=True,
                 cpu_batch=16384,
                 metric="butterfly_multiply fwd+bwd GB/s & % HBM peak, batch 16384 n=1024 fp32",
                 workload="cfg2: butterfly_multiply fw+bw, input (16384,1,1024) fp32 N(0,1), twiddle "
                          "(1,2,10,512,2,2) N(0,1/2), increasing_stride=False, grad N(0,1)"),
    "cfg3": dict(batch=8192, nstacks=1, log_n=12, nblocks=1, inc=True, cplx=True, base4=False, bw=True,
                 cpu_batch=256, autograd=True,
                 metric="butterfly_multiply fwd+bwd GB/s, complex64 FFT twiddles, batch 8192 n=4096",
                 workload="cfg3: butterfly_multiply fw+bw complex64, normalised DFT twiddles (1,1,12,2048,2,2), "
                          "input (8192,1,4096) bit-reversed outside the op, increasing_stride=True; the "
                          "butterfly_multiply operator under autograd (forward, then torch.autograd.grad)"),
    "cfg4": dict(batch=16384, nstacks=4, log_n=8, nblocks=1, inc=True, cplx=False, base4=True, bw=True,
                 cpu_batch=2048,
                 metric="butterfly_multiply_base4 fwd+bwd GB/s, batch 16384 nstacks 4 n=256 fp32",
                 workload="cfg4: butterfly_multiply_base4 fw+bw, input (16384,4,256) fp32 N(0,1), twiddle4 "
                          "(4,1,4,64,4,4) N(0,1/4), increasing_stride=True"),
    "cfg5": dict(batch=32768, nstacks=1, log_n=12, nblocks=2, inc=True, cplx=False, base4=False, bw=True,
                 cpu_batch=1024, autograd=True,
                 metric="butterfly_multiply fwd+bwd GB/s (op level), batch 32768 n=4096 fp32 nblocks 2",
                 workload="cfg5 (op level): butterfly_multiply fw+bw of Butterfly(4096, 4096, nblocks=2), input "
                          "(32768,1,4096) fp32 N(0,1), ortho twiddle (1,2,12,2048,2,2), increasing_stride=True; the "
                          "butterfly_multiply operator under autograd (forward, then torch.autograd.grad)"),
    "cfg5m": dict(batch=32768, nstacks=1, log_n=12, nblocks=2, inc=True, cplx=False, base4=False, bw=True,
                  cpu_batch=1024, module="fused",
                  metric="Butterfly(4096,4096,bias) module fwd+bwd GB/s, batch 32768 fp32 nblocks 2",
                  workload="cfg5 (module level): Butterfly(4096, 4096, bias=True, init='ortho', nblocks=2) forward + "
                           "autograd backward (d_input, d_twiddle, d_bias), input (32768,4096) fp32 N(0,1); bias "
                           "added by the kernel that writes the output, d_bias by the library's column sum"),
    "cfg5m-sep": dict(batch=32768, nstacks=1, log_n=12, nblocks=2, inc=True, cplx=False, base4=False, bw=True,
                      cpu_batch=1024, module="separate",
                      metric="Butterfly(4096,4096,bias) module fwd+bwd GB/s, bias as separate PyTorch ops",
                      workload="cfg5 (module level, unfused): the same layer computed as butterfly_multiply followed "
                               "by a PyTorch `+ bias`, autograd backward; for comparison with cfg5m"),
    "cfg3m": dict(batch=8192, nstacks=1, log_n=12, nblocks=1, inc=True, cplx=True, base4=False, bw=True,
                  cpu_batch=256, module="fft-fused",
                  metric="special.fft(4096) module fwd+bwd GB/s, complex64, batch 8192, bit reversal folded in",
                  workload="cfg3 (module level): special.fft(4096, normalized=True) = bit reversal + Butterfly, "
                           "forward + autograd backward (d_input, d_twiddle), input (8192,4096) complex64; the "
                           "bit reversal is applied by the multiply's own first read / last write"),
    "cfg3m-sep": dict(batch=8192, nstacks=1, log_n=12, nblocks=1, inc=True, cplx=True, base4=False, bw=True,
                      cpu_batch=256, module="fft-sep",
                      metric="special.fft(4096) module fwd+bwd GB/s, bit reversal as a separate gather",
                      workload="cfg3 (module level, unfused): the same two modules run one after the other "
                               "(PyTorch gather, then butterfly_multiply); for comparison with cfg3m"),
    "diag": dict(batch=16384, nstacks=1, log_n=10, nblocks=2, inc=False, cplx=False, base4=False, bw=True,
                 cpu_batch=16384, module="diag-fused",
                 metric="Diagonal-Butterfly(1024, nblocks 2)-Diagonal fwd+bwd GB/s, batch 16384 fp32, diagonals folded in",
                 workload="module level: FusedSequential(Diagonal(1024), Butterfly(1024, 1024, bias=False, nblocks=2, "
                          "increasing_stride=False), Diagonal(1024)), forward + autograd backward (d_input, "
                          "d_twiddle, both d_diagonal), input (16384,1024) fp32; the diagonals are multiplied into "
                          "the layer's first / last factor"),
    "diag-sep": dict(batch=16384, nstacks=1, log_n=10, nblocks=2, inc=False, cplx=False, base4=False, bw=True,
                     cpu_batch=16384, module="diag-sep",
                     metric="Diagonal-Butterfly(1024, nblocks 2)-Diagonal fwd+bwd GB/s, diagonals as elementwise ops",
                     workload="module level, unfused: the same three modules in a plain nn.Sequential; for "
                              "comparison with diag"),
    "legacy": dict(batch=2048, nstacks=1, log_n=9, nblocks=1, inc=True, cplx=False, base4=False, bw=True,
                   cpu_batch=2048, module="legacy",
                   metric="legacy butterfly.Butterfly(512, 512, tied_weight=False) fwd+bwd GB/s, batch 2048 fp32",
                   workload="legacy API at the shape of the reference's butterfly/benchmark.py:10-16: "
                            "Butterfly(512, 512, bias=False, tied_weight=False) (fast-format twiddle (1,9,2,512)), "
                            "input (2048,512) fp32, forward + autograd backward (d_input, d_twiddle)"),
}


def algorithmic_bytes(c):
    n = 1 << c["log_n"]
    e = 8 if c["cplx"] else 4
    row = c["nstacks"] * n * e
    twiddle = c["nstacks"] * c["nblocks"] * c["log_n"] * (n // 2) * 4 * e
    fw = 2 * row * c["batch"] + twiddle            # read input, write output, read twiddle
    bw = 3 * row * c["batch"] + 2 * twiddle        # read input + grad, write d_input; twiddle in, d_twiddle out
    return fw, (bw if c["bw"] else 0)


def algorithmic_flops(c):
    """Floating-point operations of one step, counted as the algorithm's multiply-adds (2 flops
    each): 2 per element and 2x2 stage in each sweep (4 per 4x4 stage, which stands for two),
    4 times that for complex64; sweeps = forward, and for the backward call the replay, the
    input gradient and the factor gradient."""
    n = 1 << c["log_n"]
    per_sweep = c["nstacks"] * n * c["nblocks"] * c["log_n"] * 2 * (4 if c["cplx"] else 1)
    return 2.0 * per_sweep * c["batch"] * (4 if c["bw"] else 1)


def cpu_baseline(name, c):
    """Reference csrc/cpu path (one thread) on `cpu_batch` rows of the workload, best of 3."""
    fw_b, bw_b = algorithmic_bytes(c)
    scale = c["cpu_batch"] / c["batch"]
    ref_so = os.path.join(ROOT, "oracle", "_ref", "_butterfly_ref.so")
    if os.path.isfile(ref_so) and not c["base4"]:
        out = subprocess.check_output(
            [sys.executable, os.path.join(ROOT, "oracle", "ref_runner.py"), "time", str(c["cpu_batch"]),
             str(c["nstacks"]), str(c["log_n"]), str(c["nblocks"]), str(int(c["inc"])), str(int(c["cplx"])), "3"],
            text=True)
        r = json.loads(out.strip().splitlines()[-1])
        fw_s, bw_s, kind = r["fw_s"], r["bw_s"], "reference"
    else:
        import numpy as np
        from oracle import oracle
        rng = np.random.default_rng(0)
        n, L, S, nb, B = 1 << c["log_n"], c["log_n"], c["nstacks"], c["nblocks"], c["cpu_batch"]
        dt = np.complex64 if c["cplx"] else np.float32

        def rnd(shape):
            a = rng.standard_normal(shape)
            if c["cplx"]:
                a = (a + 1j * rng.standard_normal(shape)) / math.sqrt(2)
            return a.astype(dt)

        x, g = rnd((B, S, n)), rnd((B, S, n))
        if c["base4"]:
            tw4 = (rnd((S, nb, L // 2, n // 4, 4, 4)) / 2).astype(dt)
            tw2 = (rnd((S, nb, L % 2, n // 2, 2, 2)) / math.sqrt(2)).astype(dt)
            fw = lambda: oracle.butterfly_base4_fw(tw4, tw2, x, c["inc"])
            bw = lambda: oracle.butterfly_base4_bw(tw4, tw2, x, g, c["inc"])
        else:
            tw = (rnd((S, nb, L, n // 2, 2, 2)) / math.sqrt(2)).astype(dt)
            fw = lambda: oracle.butterfly_fw(tw, x, c["inc"])
            bw = lambda: oracle.butterfly_bw(tw, x, g, c["inc"])
        fw_s = bw_s = float("inf")
        for _ in range(3):
            t0 = time.perf_counter(); fw()
            t1 = time.perf_counter()
            if c["bw"]:
                bw()
            t2 = time.perf_counter()
            fw_s, bw_s = min(fw_s, t1 - t0), min(bw_s, t2 - t1)
        kind = "port"
    total = fw_s + (bw_s if c["bw"] else 0.0)
    return {"value": (fw_b + bw_b) * scale / total / 1e9, "unit": "GB/s", "cores": 1, "kind": kind,
            "sample": f"{c['cpu_batch']} of {c['batch']} rows of the workload, best of 3 "
                      f"(fw {fw_s * 1e3:.0f} ms, bw {bw_s * 1e3:.0f} ms)",
            "rows_per_s": c["cpu_batch"] / total}


def make_operands(c, torch, dev):
    n, L, S, nb, B = 1 << c["log_n"], c["log_n"], c["nstacks"], c["nblocks"], c["batch"]
    dtype = torch.complex64 if c["cplx"] else torch.float32
    if c["base4"]:
        tw4 = (torch.randn(S, nb, L // 2, n // 4, 4, 4, dtype=dtype) / 2).to(dev)
        tw2 = (torch.randn(S, nb, L % 2, n // 2, 2, 2, dtype=dtype) / 2 ** 0.5).to(dev)
        tws = (tw4, tw2)
    elif c["cplx"] and S == 1 and nb == 1:
        from butterfly_amd import special
        tws = (special.fft(n, normalized=True, with_br_perm=False).twiddle.detach().to(dev),)
    elif nb == 2 and L == 12 and not c["cplx"]:
        import butterfly_amd
        tws = (butterfly_amd.Butterfly(n, n, bias=True, init="ortho", nblocks=2).twiddle.detach().to(dev),)
    else:
        tws = ((torch.randn(S, nb, L, n // 2, 2, 2, dtype=dtype) / 2 ** 0.5).to(dev),)
    x = torch.randn(B, S, n, dtype=dtype).to(dev)
    grad = torch.randn(B, S, n, dtype=dtype).to(dev)
    return tws, x, grad


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", default="cfg2", choices=sorted(CONFIGS))
    ap.add_argument("--shape", default=None, metavar="B,S,LOG_N,NBLOCKS,f32|c64[,inc|dec]",
                    help="forward + backward at an arbitrary shape instead of a named configuration")
    ap.add_argument("--batch", type=int, default=None, help="run the configuration at another batch size")
    ap.add_argument("--settle-ms", type=float, default=250.0,
                    help="run untimed steps for this long before the warmup steps: the GPU raises its clocks "
                         "over the first tens of milliseconds of sustained load, and kernels launched in that "
                         "window run 10-20 %% slower than in steady state")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--graph", action="store_true",
                    help="record the step (forward + backward) once with butterfly_amd.GraphedStep and time its "
                         "replays: what a caller with fixed shapes pays per step at small batch")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run plain device copies of the input (a kernel of known traffic, for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU; --gpus must be 1 (the rows of a batch would shard across GPUs; only d_twiddle would need a reduction)")
    c = CONFIGS[args.config]
    if args.shape:
        f = args.shape.split(",")
        B, S, L, nb = (int(v) for v in f[:4])
        cplx = f[4] == "c64"
        inc = len(f) < 6 or f[5] == "inc"
        args.config = "shape"
        c = dict(batch=B, nstacks=S, log_n=L, nblocks=nb, inc=inc, cplx=cplx, base4=False, bw=True,
                 cpu_batch=max(1, min(B, (1 << 21) // (S << L))),
                 metric=f"butterfly_multiply fwd+bwd GB/s, batch {B} nstacks {S} n={1 << L} nblocks {nb} "
                        f"{'complex64' if cplx else 'fp32'}",
                 workload=f"shape: butterfly_multiply fw+bw, input ({B},{S},{1 << L}) {'complex64' if cplx else 'fp32'} "
                          f"N(0,1), twiddle ({S},{nb},{L},{(1 << L) // 2},2,2) N(0,1/2), increasing_stride={inc}")

    if args.batch is not None:
        c = dict(c, batch=args.batch, cpu_batch=min(c["cpu_batch"], args.batch),
                 metric=c["metric"] + f" [batch overridden: {args.batch}]",
                 workload=c["workload"] + f" [batch overridden: {args.batch}]")

    import torch
    import butterfly_amd
    ops = torch.ops.torch_butterfly
    assert torch.cuda.is_available(), "bench.py needs a HIP device"
    torch.manual_seed(0)
    dev = torch.device("cuda:0")
    tws, x, grad = make_operands(c, torch, dev)
    inc = c["inc"]

    if c.get("module", "").startswith("fft"):
        # module level: bit reversal + butterfly, then autograd for both gradients
        from butterfly_amd import special
        layer = special.fft(1 << c["log_n"], normalized=True).to(dev)
        if c["module"] == "fft-sep":
            layer = torch.nn.Sequential(*layer)
        xm = x.reshape(c["batch"], -1).requires_grad_()
        gm = grad.reshape(c["batch"], -1)
        state = {}

        def fw_call():
            state["y"] = layer(xm)
        bw_call = lambda: torch.autograd.grad(state["y"], (xm, layer[1].twiddle), gm)
    elif c.get("module", "").startswith("diag"):
        from butterfly_amd.diagonal import Diagonal
        from butterfly_amd.permutation import FusedSequential
        n = 1 << c["log_n"]
        layer = FusedSequential(Diagonal(n), butterfly_amd.Butterfly(n, n, bias=False, nblocks=c["nblocks"],
                                                                     increasing_stride=c["inc"]), Diagonal(n)).to(dev)
        if c["module"] == "diag-sep":
            layer = torch.nn.Sequential(*layer)
        xm = x.reshape(c["batch"], -1).requires_grad_()
        gm = grad.reshape(c["batch"], -1)
        params = [xm] + list(layer.parameters())
        state = {}

        def fw_call():
            state["y"] = layer(xm)
        bw_call = lambda: torch.autograd.grad(state["y"], params, gm)
    elif c.get("module") == "legacy":
        from butterfly_amd import legacy
        layer = legacy.Butterfly(1 << c["log_n"], 1 << c["log_n"], bias=False, tied_weight=False).to(dev)
        xm = x.reshape(c["batch"], -1).requires_grad_()
        gm = grad.reshape(c["batch"], -1)
        state = {}

        def fw_call():
            state["y"] = layer(xm)
        bw_call = lambda: torch.autograd.grad(state["y"], (xm, layer.twiddle), gm)
    elif c.get("module"):
        # module level: the layer's forward, then autograd for all three gradients
        layer = butterfly_amd.Butterfly(1 << c["log_n"], 1 << c["log_n"], bias=True, init="ortho",
                                        nblocks=c["nblocks"]).to(dev)
        xm = x.reshape(c["batch"], -1).requires_grad_()
        gm = grad.reshape(c["batch"], -1)
        state = {}
        if c["module"] == "fused":
            def fw_call():
                state["y"] = layer(xm)
        else:
            from butterfly_amd.multiply import butterfly_multiply

            def fw_call():
                z = butterfly_multiply(layer.twiddle, layer.pre_process(xm), layer.increasing_stride, layer.out_size)
                state["y"] = z.reshape(c["batch"], -1) + layer.bias
        bw_call = lambda: torch.autograd.grad(state["y"], (xm, layer.twiddle, layer.bias), gm)
    elif c["base4"]:
        fw_call = lambda: ops.butterfly_multiply_base4_fw(tws[0], tws[1], x, inc, None)
        bw_call = lambda: ops.butterfly_multiply_base4_bw(tws[0], tws[1], x, grad, inc)
    elif c.get("autograd"):
        # the differentiable operator, as a training step calls it: its forward keeps what a backward
        # in several passes would otherwise recompute
        twg, xg = tws[0].requires_grad_(), x.requires_grad_()
        state = {}

        def fw_call():
            state["y"] = ops.butterfly_multiply(twg, xg, inc, None)
        bw_call = lambda: torch.autograd.grad(state["y"], (twg, xg), grad)
    else:
        fw_call = lambda: ops.butterfly_multiply_fw(tws[0], x, inc, None)
        bw_call = lambda: ops.butterfly_multiply_bw(tws[0], x, grad, inc)

    if args.graph:
        # the whole step recorded once with the helper the package offers; a replay is one launch, so
        # there is one interval per step
        if c.get("module"):
            wrt = [t for t in layer.parameters() if t.requires_grad]
            fn, x_rec, g_rec = layer, xm.detach(), gm
        elif c["base4"]:
            wrt = [t.requires_grad_() for t in tws if t.numel()]
            fn = lambda t: ops.butterfly_multiply_base4(tws[0], tws[1], t, inc, None)
            x_rec, g_rec = x, grad
        else:
            wrt = [tws[0].requires_grad_()]
            fn = lambda t: ops.butterfly_multiply(tws[0], t, inc, None)
            x_rec, g_rec = x, grad
        recorded = butterfly_amd.GraphedStep(fn, x_rec, g_rec if c["bw"] else None, wrt if c["bw"] else ())
        fw_call = recorded.replay
        c = dict(c, bw=False, graphed_bw=c["bw"], metric=c["metric"] + " [step replayed from a HIP graph]",
                 workload=c["workload"] + " [forward" + (" + backward" if c["bw"] else "") + " recorded once with "
                          "GraphedStep, each step one replay]")

    def untimed_step():
        fw_call()
        if c["bw"]:
            bw_call()

    settle_t0 = time.perf_counter()
    while (time.perf_counter() - settle_t0) * 1e3 < args.settle_ms:
        for _ in range(4):
            untimed_step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        untimed_step()
    torch.cuda.synchronize()
    if args.calibrate_copy:
        dst = torch.empty_like(x)
        for _ in range(5):
            dst.copy_(x)
        torch.cuda.synchronize()
    # Two timed regions of K steps each.  The first has nothing in it but the steps, bracketed by
    # device synchronisation and the host clock: `value` and `ms_per_step` come from it (an event
    # record costs the host several microseconds and the device a signal packet between two
    # kernels, which is a third of a step at the small configurations).  The second repeats the K
    # steps with one device event between consecutive calls (the end of a call is the start of the
    # next one) and gives the split into forward and backward call that `roofline` is priced on.
    per_step = 2 if c["bw"] else 1
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        fw_call()
        if c["bw"]:
            bw_call()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(per_step * args.steps + 1)]
    torch.cuda.synchronize()
    marks[0].record()
    for i in range(args.steps):
        fw_call()
        marks[per_step * i + 1].record()
        if c["bw"]:
            bw_call()
            marks[per_step * i + 2].record()
    torch.cuda.synchronize()
    span = lambda j: marks[j].elapsed_time(marks[j + 1])
    fw_ms = sum(span(per_step * i) for i in range(args.steps)) / args.steps
    bw_ms = sum(span(per_step * i + 1) for i in range(args.steps)) / args.steps if c["bw"] else 0.0
    ms_per_step = wall * 1e3 / args.steps
    fw_b, bw_b = algorithmic_bytes(dict(c, bw=c["bw"] or c.get("graphed_bw", False)))
    value = (fw_b + bw_b) / (ms_per_step * 1e-3) / 1e9
    if c["bw"]:
        dom_name, dom_b, dom_ms = "backward call (all its launches incl. the partial-sum reduce)", bw_b, bw_ms
    else:
        dom_name, dom_b, dom_ms = ("recorded step" if args.graph else "forward call"), fw_b + bw_b, fw_ms
    dom_gbs = dom_b / (dom_ms * 1e-3) / 1e9
    line = {
        "metric": c["metric"], "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "settle_ms": args.settle_ms, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "c64" if c["cplx"] else "f32", "data": "synthetic",
        "config": {"workload": c["workload"]},
        "pct_hbm_peak": 100.0 * value / HBM_PEAK_GBS,
        "rows_per_s": c["batch"] / (ms_per_step * 1e-3),
        "fw_ms": fw_ms, "bw_ms": bw_ms,
        "fw_GBps": fw_b / (fw_ms * 1e-3) / 1e9,
        "roofline": {"bound": "hbm", "kernel": dom_name, "achieved": dom_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": dom_gbs / HBM_PEAK_GBS,
                     "traffic": None if args.graph else measured_traffic(args.config)},
        "graphed": bool(args.graph),
    }
    # the dominant kernel by itself, from the committed kernel-trace summary of this same command
    # (its average launch duration and the algorithmic bytes of one launch)
    kern = None if args.graph else measured_kernel(args.config)
    if kern:
        line["roofline"].update({"kernel_name": kern[0], "kernel_us": kern[1], "kernel_bytes": kern[2],
                                 "frac_kernel": kern[2] / (kern[1] * 1e-6) / 1e9 / HBM_PEAK_GBS})
    # second roofline of the path: the same step against the fp32 vector rate (no MFMA: the
    # factors are 2x2 / 4x4 blocks, not a dense contraction)
    flops = algorithmic_flops(dict(c, bw=c["bw"] or c.get("graphed_bw", False)))
    tflops = flops / (ms_per_step * 1e-3) / 1e12
    line["valu"] = {"achieved": tflops, "peak": VALU_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tflops / VALU_PEAK_TFLOPS,
                    "flops_per_step": flops}
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(args.config, c)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
