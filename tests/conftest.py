import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (MI355X)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no HIP device")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def randn(rng, shape, dtype):
    """Standard normal samples; complex dtypes get variance 1/2 per component."""
    dtype = np.dtype(dtype)
    if dtype.kind == "c":
        return ((rng.standard_normal(shape) + 1j * rng.standard_normal(shape)) / np.sqrt(2)).astype(dtype)
    return rng.standard_normal(shape).astype(dtype)


def rel_err(a, b):
    """max |a - b| / max |b| -- the error measure the tolerances in these tests refer to."""
    a, b = np.asarray(a), np.asarray(b)
    assert a.shape == b.shape, (a.shape, b.shape)
    if b.size == 0:
        return 0.0
    scale = np.abs(b).max()
    return float(np.abs(a - b).max() / (scale if scale > 0 else 1.0))


def dense_stage2(n, log_stride, tw):
    """Dense n x n matrix of one base-2 stage; tw is (n/2, 2, 2)."""
    st = 1 << log_stride
    M = np.zeros((n, n), dtype=tw.dtype)
    for i in range(n // 2):
        low = i % st
        pos = 2 * (i - low) + low
        for r in range(2):
            for c in range(2):
                M[pos + r * st, pos + c * st] = tw[i, r, c]
    return M


def dense_stage4(n, log_stride, tw):
    """Dense matrix of one radix-4 stage; tw is (n/4, 4, 4)."""
    st = 1 << log_stride
    M = np.zeros((n, n), dtype=tw.dtype)
    for q in range(n // 4):
        low = q % st
        pos = 4 * (q - low) + low
        for r in range(4):
            for c in range(4):
                M[pos + r * st, pos + c * st] = tw[q, r, c]
    return M


def dense_butterfly(twiddle_s, increasing_stride):
    """Dense matrix of a whole base-2 product for one stack: twiddle_s is (nb, L, n/2, 2, 2)."""
    nb, L = twiddle_s.shape[:2]
    n = 1 << L
    M = np.eye(n, dtype=twiddle_s.dtype)
    for block in range(nb):
        inc = bool(increasing_stride) != bool(block % 2)
        for idx in range(L):
            ls = idx if inc else L - 1 - idx
            M = dense_stage2(n, ls, twiddle_s[block, idx]) @ M
    return M
