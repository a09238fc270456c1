"""Device-event timing helpers (counterpart of torch_butterfly/benchmark_utils.py:7-28)."""
import numpy as np
import torch


def benchmark(fn, nrepeats=7):
    """Median and standard deviation, in seconds, of ``fn()`` timed with device events."""
    fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(nrepeats):
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        end.record()
        torch.cuda.synchronize()
        times.append(start.elapsed_time(end) / 1000)
    return float(np.median(times)), float(np.std(times))


def benchmark_fw_bw(fn, inputs, nrepeats=7):
    """(median, std) of forward, backward and forward+backward of ``fn(*inputs)``."""
    def forward():
        return fn(*inputs)

    out = forward()
    grad = torch.randn_like(out)
    params = [t for t in inputs if isinstance(t, torch.Tensor) and t.requires_grad]

    def backward():
        return torch.autograd.grad(out, params, grad, retain_graph=True)

    def both():
        return torch.autograd.grad(fn(*inputs), params, grad)

    return benchmark(forward, nrepeats), benchmark(backward, nrepeats), benchmark(both, nrepeats)
