"""Functional entry points of the base-2 butterfly multiply.

``butterfly_multiply{,_fw,_bw}`` call the registered operators (HIP kernels for device tensors;
host tensors run on the operators' single-threaded host path, as the reference's run on its
csrc/cpu); they are the counterparts of the scripted wrappers in the reference's
torch_butterfly/multiply.py:8-25.  The operators that are new here (bias and permutations
folded in) exist for device tensors only: for host tensors the wrappers below compose them
from butterfly_multiply and plain tensor operations.
``butterfly_multiply_torch`` is a plain-PyTorch restatement of the same product, kept as a
differentiable cross-check like the reference's (multiply.py:28-51); nothing dispatches to
it automatically.
"""
from typing import Optional, Tuple

import torch


def butterfly_multiply_fw(twiddle: torch.Tensor, input: torch.Tensor, increasing_stride: bool,
                          output_size: Optional[int] = None) -> torch.Tensor:
    return torch.ops.torch_butterfly.butterfly_multiply_fw(twiddle, input, increasing_stride,
                                                           output_size)


def butterfly_multiply_bw(twiddle: torch.Tensor, input: torch.Tensor, grad: torch.Tensor,
                          increasing_stride: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    return torch.ops.torch_butterfly.butterfly_multiply_bw(twiddle, input, grad, increasing_stride)


def butterfly_multiply(twiddle: torch.Tensor, input: torch.Tensor, increasing_stride: bool,
                       output_size: Optional[int] = None) -> torch.Tensor:
    """twiddle (nstacks, nblocks, log_n, n/2, 2, 2); input (batch, nstacks, input_size), zero
    padded or trimmed to n; returns (batch, nstacks, output_size or n).  Differentiable."""
    return torch.ops.torch_butterfly.butterfly_multiply(twiddle, input, increasing_stride,
                                                        output_size)


def butterfly_multiply_bias(twiddle: torch.Tensor, input: torch.Tensor, bias: torch.Tensor,
                            increasing_stride: bool, output_size: Optional[int] = None) -> torch.Tensor:
    """butterfly_multiply(...) + bias with the addition done by the kernel that writes the
    output; bias (nstacks, output_size or n).  Differentiable in all three tensors.  The
    reference adds the bias as a separate pass (torch_butterfly/butterfly.py:152-169)."""
    if not input.is_cuda:
        return butterfly_multiply(twiddle, input, increasing_stride, output_size) + bias
    return torch.ops.torch_butterfly.butterfly_multiply_bias(twiddle, input, bias, increasing_stride,
                                                             output_size)


def butterfly_multiply_perm(twiddle: torch.Tensor, input: torch.Tensor, in_perm: Optional[torch.Tensor],
                            out_index: Optional[torch.Tensor], bias: Optional[torch.Tensor],
                            increasing_stride: bool, output_size: Optional[int] = None) -> torch.Tensor:
    """The multiply between two fixed column permutations that the kernels fold into their
    first read and last write: u[..., c] = input[..., in_perm[c]], y = multiply(u) + bias,
    output[..., out_index[c]] = y[..., c].  Tables are int32 of n entries (None = identity); a
    FixedPermutation(q) behind the layer is out_index = inverse of q.  Differentiable in
    twiddle, input and bias.  The reference runs each permutation as a separate gather
    (torch_butterfly/permutation.py:55-78)."""
    if not input.is_cuda:
        n = 1 << twiddle.shape[2]   # (not 2 * pairs: a layer of size 1 has no pairs)
        cols = n if output_size is None else output_size
        x = input
        if in_perm is not None:
            x = fit_last_dim(x, n).index_select(-1, in_perm.long())
        y = butterfly_multiply(twiddle, x, increasing_stride, None)
        if bias is not None:
            y = y + torch.nn.functional.pad(bias, (0, n - cols))
        if out_index is not None:
            y = torch.zeros_like(y).index_copy(-1, out_index.long(), y)
        return y[..., :cols]
    return torch.ops.torch_butterfly.butterfly_multiply_perm(twiddle, input, in_perm, out_index, bias,
                                                             increasing_stride, output_size)


def fit_last_dim(x: torch.Tensor, n: int) -> torch.Tensor:
    """Zero-pad or trim the last dimension to exactly ``n``."""
    size = x.shape[-1]
    if size == n:
        return x
    if size > n:
        return x[..., :n]
    return torch.nn.functional.pad(x, (0, n - size))


def stage_strides(log_n: int, nblocks: int, increasing_stride: bool):
    """log2(stride) of every stage, block by block (direction alternates per block)."""
    out = []
    for block in range(nblocks):
        inc = increasing_stride != (block % 2 == 1)
        out.append([idx if inc else log_n - 1 - idx for idx in range(log_n)])
    return out


def butterfly_multiply_torch(twiddle, input, increasing_stride=True, output_size=None):
    batch, nstacks, _ = input.shape
    nblocks, log_n = twiddle.shape[1], twiddle.shape[2]
    n = 1 << log_n
    if tuple(twiddle.shape) != (nstacks, nblocks, log_n, n // 2, 2, 2):
        raise ValueError("twiddle must have shape (nstacks, nblocks, log_n, n / 2, 2, 2)")
    output_size = n if output_size is None else output_size
    if output_size > n:
        raise ValueError("output_size must be <= n")
    x = fit_last_dim(input, n)
    for block, strides in enumerate(stage_strides(log_n, nblocks, increasing_stride)):
        for idx, log_stride in enumerate(strides):
            st = 1 << log_stride
            # pair i = h * st + l couples elements (2 h st + l) and (2 h st + st + l)
            t = twiddle[:, block, idx].reshape(nstacks, n // (2 * st), st, 2, 2)
            xv = x.reshape(batch, nstacks, n // (2 * st), 2, st)
            x = torch.einsum("shlrc,bshcl->bshrl", t, xv).reshape(batch, nstacks, n)
    return x[:, :, :output_size]
