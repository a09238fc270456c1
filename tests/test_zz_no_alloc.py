"""The backward entry point that allocates nothing (bf_butterfly_multiply_bw_noalloc): its
results against bf_butterfly_multiply_bw (same kernels, same launch plan: identical bits) and
against the CPU oracle, on two calls in a row that share the library's built-in scratch area,
the second on a smaller input."""
import sys

import numpy as np
import pytest
import torch

from conftest import randn, rel_err
from oracle import oracle

pytestmark = pytest.mark.gpu

BW_TOL = 1e-4


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def operands(rng, dtype, B, S, L, nb, I=None, O=None):
    n = 1 << L
    tw = (randn(rng, (S, nb, L, n // 2, 2, 2), dtype) / np.sqrt(2)).astype(dtype)
    return tw, randn(rng, (B, S, n if I is None else I), dtype), randn(rng, (B, S, n if O is None else O), dtype)


def run_pair(tw, x, g, inc):
    from butterfly_amd import _capi
    twd, xd, gd = dev(tw), dev(x), dev(g)
    # results allocated before the call: the call itself must not need the allocator
    dtw = torch.full_like(twd, float("nan"))
    dx = torch.full(xd.shape, float("nan"), dtype=xd.dtype, device=xd.device)
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    # PyTorch's statistics see its own allocator only; the device's free memory also sees a
    # hipMalloc made inside the library
    # (one call first: the runtime loads a kernel's code on its first launch, which is not the
    # library allocating)
    _capi.multiply_bw_noalloc(twd, xd, gd, inc, dtw, dx)
    torch.cuda.synchronize()
    dtw.fill_(float("nan"))
    dx.fill_(float("nan"))
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    free_before = torch.cuda.mem_get_info()[0]
    _capi.multiply_bw_noalloc(twd, xd, gd, inc, dtw, dx)
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
    assert torch.cuda.mem_get_info()[0] == free_before
    ref_dtw, ref_dx = _capi.multiply_bw(twd, xd, gd, inc)
    torch.cuda.synchronize()
    assert torch.equal(dtw, ref_dtw) and torch.equal(dx, ref_dx)
    o_dtw, o_dx = oracle.butterfly_bw(tw, x, g, inc)
    assert rel_err(dx.cpu().numpy(), o_dx) < BW_TOL
    assert rel_err(dtw.cpu().numpy(), o_dtw) < BW_TOL


@pytest.mark.parametrize("dtype", [np.float32, np.complex64], ids=["f32", "c64"])
def test_two_calls_in_a_row_share_the_scratch_area(dtype):
    rng = np.random.default_rng(9100)
    # first call: many workgroups, two blocks -> a wide use of the area (complex64 needs twice
    # the bytes per partial slice plus an activation between its two passes: fewer rows)
    say("noalloc first call", np.dtype(dtype).name)
    run_pair(*operands(rng, dtype, 3000 if dtype is np.float32 else 200, 1, 10, 2), False)
    # second call, smaller in every way: fewer slices, shorter rows, padded input, trimmed output
    say("noalloc second call", np.dtype(dtype).name)
    run_pair(*operands(rng, dtype, 37, 2, 7, 1, I=100, O=90), True)
    # a schedule of several launches (activations between the passes also live in the area)
    say("noalloc third call", np.dtype(dtype).name)
    run_pair(*operands(rng, dtype, 50, 1, 12, 2), True)


def test_headline_shape_fits_and_oversized_problems_are_refused():
    from butterfly_amd import _capi
    rng = np.random.default_rng(9101)
    tw, x, g = operands(rng, np.float32, 16384, 1, 10, 2)
    say("noalloc headline")
    twd, xd, gd = dev(tw), dev(x), dev(g)
    dtw, dx = _capi.multiply_bw_noalloc(twd, xd, gd, False)
    ref_dtw, ref_dx = _capi.multiply_bw(twd, xd, gd, False)
    assert torch.equal(dtw, ref_dtw) and torch.equal(dx, ref_dx)
    # (8192, 1, 4096) needs two (B, S, n) activations between its passes: 256 MiB
    say("noalloc oversized")
    tw, x, g = operands(rng, np.float32, 8192, 1, 12, 1)
    with pytest.raises(_capi.ButterflyError, match="built-in area") as e:
        _capi.multiply_bw_noalloc(dev(tw), dev(x), dev(g), True)
    assert e.value.code == -4
