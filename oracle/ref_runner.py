"""Run the compiled reference operators in a process of their own (TEST INFRASTRUCTURE ONLY).

``oracle/_ref/_butterfly_ref.so`` registers the same ``torch_butterfly`` operator
namespace as the product library, and the dispatcher allows one registration per
process, so the reference build is always driven through this script:

    python oracle/ref_runner.py run  cases_in.npz cases_out.npz
    python oracle/ref_runner.py time <batch> <nstacks> <log_n> <nblocks> <inc> <complex> <reps>

``run``: the input archive holds, for every case ``i``, ``c{i}_twiddle``, ``c{i}_input``,
optionally ``c{i}_grad``, and ``c{i}_meta = [increasing_stride, output_size or -1]``.  The
output archive holds ``c{i}_output`` and, when a gradient was given, ``c{i}_d_twiddle``
and ``c{i}_d_input``.

``time``: prints one JSON line with the best-of-``reps`` wall time of fw and bw on
seeded random operands (single thread, like the reference).
"""
import json
import os
import sys
import time

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REF_SO = os.path.join(HERE, "_ref", "_butterfly_ref.so")


def load():
    torch.ops.load_library(REF_SO)
    return torch.ops.torch_butterfly


def run(inp, outp):
    ops = load()
    data = np.load(inp)
    ncases = len([k for k in data.files if k.endswith("_meta")])
    out = {}
    for i in range(ncases):
        tw = torch.from_numpy(data[f"c{i}_twiddle"])
        x = torch.from_numpy(data[f"c{i}_input"])
        inc, osz = [int(v) for v in data[f"c{i}_meta"]]
        y = ops.butterfly_multiply_fw(tw, x, bool(inc), None if osz < 0 else osz)
        out[f"c{i}_output"] = y.contiguous().numpy()
        if f"c{i}_grad" in data.files:
            g = torch.from_numpy(data[f"c{i}_grad"])
            dtw, dx = ops.butterfly_multiply_bw(tw, x, g, bool(inc))
            out[f"c{i}_d_twiddle"] = dtw.contiguous().numpy()
            out[f"c{i}_d_input"] = dx.contiguous().numpy()
    np.savez(outp, **out)


def timeit(batch, nstacks, log_n, nblocks, inc, cplx, reps):
    ops = load()
    torch.set_num_threads(1)
    n = 1 << log_n
    dtype = torch.complex64 if cplx else torch.float32
    g = torch.Generator().manual_seed(0)
    tw = torch.randn(nstacks, nblocks, log_n, n // 2, 2, 2, dtype=dtype, generator=g) / (2 ** 0.5)
    x = torch.randn(batch, nstacks, n, dtype=dtype, generator=g)
    grad = torch.randn(batch, nstacks, n, dtype=dtype, generator=g)
    ops.butterfly_multiply_fw(tw, x[:8], bool(inc), None)
    fw = bw = float("inf")
    for _ in range(reps):
        t0 = time.perf_counter()
        ops.butterfly_multiply_fw(tw, x, bool(inc), None)
        t1 = time.perf_counter()
        ops.butterfly_multiply_bw(tw, x, grad, bool(inc))
        t2 = time.perf_counter()
        fw, bw = min(fw, t1 - t0), min(bw, t2 - t1)
    print(json.dumps({"fw_s": fw, "bw_s": bw, "batch": batch, "threads": 1}))


if __name__ == "__main__":
    if sys.argv[1] == "run":
        run(sys.argv[2], sys.argv[3])
    elif sys.argv[1] == "time":
        timeit(*[int(v) for v in sys.argv[2:9]])
    else:
        raise SystemExit(__doc__)
