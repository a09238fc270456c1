"""Base-4 butterfly multiply: radix-4 stages (4x4 factors on quads) plus one 2x2 stage when
log_n is odd.

``butterfly_multiply_base4`` calls the native operators (new in this library; the
reference computes the same product with PyTorch views in
torch_butterfly/multiply_base4.py:7-41).  ``butterfly_multiply_base4_torch`` is a
plain-PyTorch restatement for cross-checks and ``twiddle_base2_to_base4`` fuses pairs of
base-2 stages into base-4 factors (multiply_base4.py:44-71).
"""
from typing import Optional

import torch

from .multiply import fit_last_dim


def butterfly_multiply_base4_fw(twiddle4, twiddle2, input, increasing_stride: bool,
                                output_size: Optional[int] = None):
    return torch.ops.torch_butterfly.butterfly_multiply_base4_fw(twiddle4, twiddle2, input,
                                                                 increasing_stride, output_size)


def butterfly_multiply_base4_bw(twiddle4, twiddle2, input, grad, increasing_stride: bool):
    return torch.ops.torch_butterfly.butterfly_multiply_base4_bw(twiddle4, twiddle2, input, grad,
                                                                 increasing_stride)


def butterfly_multiply_base4(twiddle4, twiddle2, input, increasing_stride: bool = True,
                             output_size: Optional[int] = None):
    """twiddle4 (nstacks, nblocks, log_n // 2, n/4, 4, 4); twiddle2 (nstacks, nblocks,
    log_n % 2, n/2, 2, 2); input (batch, nstacks, input_size).  Differentiable.  Host tensors
    take the PyTorch formulation below, which is the reference's only base-4 path
    (torch_butterfly/multiply_base4.py:7-41); the native operators are for device tensors."""
    if not input.is_cuda:
        return butterfly_multiply_base4_torch(twiddle4, twiddle2, input, increasing_stride, output_size)
    return torch.ops.torch_butterfly.butterfly_multiply_base4(twiddle4, twiddle2, input,
                                                              increasing_stride, output_size)


def _base4_log_n(twiddle4, twiddle2):
    return twiddle4.shape[2] * 2 + twiddle2.shape[2]


def butterfly_multiply_base4_torch(twiddle4, twiddle2, input, increasing_stride=True,
                                   output_size=None):
    batch, nstacks, _ = input.shape
    nblocks = twiddle4.shape[1]
    log_n = _base4_log_n(twiddle4, twiddle2)
    n = 1 << log_n
    if log_n >= 2 and tuple(twiddle4.shape) != (nstacks, nblocks, log_n // 2, n // 4, 4, 4):
        raise ValueError("twiddle4 must have shape (nstacks, nblocks, log_n // 2, n / 4, 4, 4)")
    if log_n % 2 == 1 and tuple(twiddle2.shape) != (nstacks, nblocks, 1, n // 2, 2, 2):
        raise ValueError("twiddle2 must have shape (nstacks, nblocks, 1, n / 2, 2, 2)")
    output_size = n if output_size is None else output_size
    if output_size > n:
        raise ValueError("output_size must be <= n")
    x = fit_last_dim(input, n)
    for block in range(nblocks):
        inc = increasing_stride != (block % 2 == 1)
        for idx in range(log_n // 2):
            st = 1 << (2 * idx if inc else log_n - 2 - 2 * idx)
            t = twiddle4[:, block, idx].reshape(nstacks, n // (4 * st), st, 4, 4)
            xv = x.reshape(batch, nstacks, n // (4 * st), 4, st)
            x = torch.einsum("shlrc,bshcl->bshrl", t, xv).reshape(batch, nstacks, n)
        if log_n % 2 == 1:
            st = (n // 2) if inc else 1
            t = twiddle2[:, block, 0].reshape(nstacks, n // (2 * st), st, 2, 2)
            xv = x.reshape(batch, nstacks, n // (2 * st), 2, st)
            x = torch.einsum("shlrc,bshcl->bshrl", t, xv).reshape(batch, nstacks, n)
    return x[:, :, :output_size]


def twiddle_base2_to_base4(twiddle, increasing_stride=True):
    """Fuse base-2 stages (2 idx, 2 idx + 1) of every block into one 4x4 factor per quad.

    With radix-4 stride st, quad q = h st + l holds the elements 4 h st + l + c st, c = 2a + b.
    One of the fused stages pairs along b (stride st, pair index (2h + a) st + l), the other
    along a (stride 2 st, pair index 2 h st + b st + l); the 4x4 factor is their product in
    execution order.  Returns (twiddle4, twiddle2) with twiddle2 the leftover last stage when
    log_n is odd, else an empty (nstacks, nblocks, 0, n/2, 2, 2) tensor.
    """
    nstacks, nblocks, log_n = twiddle.shape[:3]
    n = 1 << log_n
    if tuple(twiddle.shape) != (nstacks, nblocks, log_n, n // 2, 2, 2):
        raise ValueError("twiddle must have shape (nstacks, nblocks, log_n, n / 2, 2, 2)")
    if log_n % 2 == 1:
        twiddle2 = twiddle[:, :, -1:]
    else:
        twiddle2 = twiddle.new_empty(nstacks, nblocks, 0, n // 2, 2, 2)
    twiddle4 = twiddle.new_empty(nstacks, nblocks, log_n // 2, n // 4, 4, 4)
    for block in range(nblocks):
        inc = increasing_stride != (block % 2 == 1)
        for idx in range(log_n // 2):
            st = 1 << (2 * idx if inc else log_n - 2 - 2 * idx)
            shape = (nstacks, n // (4 * st), 2, st, 2, 2)
            first = twiddle[:, block, 2 * idx].reshape(shape)
            second = twiddle[:, block, 2 * idx + 1].reshape(shape)
            if inc:
                # first pairs along b (indexed by a), second pairs along a (indexed by b)
                fused = torch.einsum("shblax,shxlby->shlabxy", second, first)
            else:
                # first pairs along a (indexed by b), second pairs along b (indexed by a)
                fused = torch.einsum("shalby,shylax->shlabxy", second, first)
            twiddle4[:, block, idx] = fused.reshape(nstacks, n // 4, 4, 4)
    return twiddle4, twiddle2
