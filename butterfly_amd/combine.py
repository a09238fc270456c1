"""Twiddle algebra: fold a diagonal into a Butterfly, concatenate two Butterflies
(reference: torch_butterfly/combine.py:11-80)."""
import copy

import torch
from torch.nn import functional as F

from .butterfly import Butterfly


def diagonal_butterfly(butterfly: Butterfly, diagonal: torch.Tensor, diag_first: bool,
                       inplace: bool = True) -> Butterfly:
    """Butterfly equal to ``butterfly @ diag`` (diag_first) or ``diag @ butterfly``.

    The diagonal scales the columns of the first stage (whose pairs are (2i, 2i+1) for
    increasing stride and (i, i + n/2) for decreasing) or the rows of the last stage.
    nstacks must be 1 and there must be no bias."""
    if butterfly.nstacks != 1 or butterfly.bias is not None:
        raise ValueError("diagonal_butterfly needs nstacks == 1 and no bias")
    twiddle = butterfly.twiddle.detach().clone()
    n = 1 << twiddle.shape[2]
    if diagonal.shape[-1] < n:
        diagonal = F.pad(diagonal, (0, n - diagonal.shape[-1]), value=1)
    adjacent = (diagonal[0::2], diagonal[1::2])
    halves = (diagonal[:n // 2], diagonal[n // 2:])
    if diag_first:
        lo, hi = adjacent if butterfly.increasing_stride else halves
        twiddle[:, 0, 0, :, :, 0] *= lo.unsqueeze(-1)
        twiddle[:, 0, 0, :, :, 1] *= hi.unsqueeze(-1)
    else:
        last_inc = butterfly.increasing_stride != ((butterfly.nblocks - 1) % 2 == 1)
        lo, hi = halves if last_inc else adjacent
        twiddle[:, -1, -1, :, 0, :] *= lo.unsqueeze(-1)
        twiddle[:, -1, -1, :, 1, :] *= hi.unsqueeze(-1)
    out = butterfly if inplace else copy.deepcopy(butterfly)
    with torch.no_grad():
        out.twiddle.copy_(twiddle)
    return out


def butterfly_product(butterfly1: Butterfly, butterfly2: Butterfly) -> Butterfly:
    """One Butterfly computing ``butterfly2(butterfly1(x))`` (blocks concatenated; an identity
    block is inserted when the stride directions would not alternate)."""
    if butterfly1.bias is not None or butterfly2.bias is not None:
        raise ValueError("butterfly_product needs bias-free factors")
    if (butterfly1.complex != butterfly2.complex or butterfly1.nstacks != butterfly2.nstacks
            or butterfly1.log_n != butterfly2.log_n):
        raise ValueError("factors must agree in dtype kind, nstacks and log_n")
    next_inc = butterfly1.increasing_stride != (butterfly1.nblocks % 2 == 1)
    if next_inc != butterfly2.increasing_stride:
        eye = Butterfly(butterfly1.in_size, butterfly1.out_size, bias=False, complex=butterfly1.complex,
                        increasing_stride=next_inc, init="identity").to(butterfly1.twiddle.device)
        butterfly1 = butterfly_product(butterfly1, eye)
    twiddle = torch.cat((butterfly1.twiddle.detach(), butterfly2.twiddle.detach()), dim=1)
    n = 1 << butterfly1.log_n
    out = Butterfly(n, n, bias=False, complex=butterfly1.complex,
                    increasing_stride=butterfly1.increasing_stride, init=twiddle,
                    nblocks=butterfly1.nblocks + butterfly2.nblocks)
    out.in_size = butterfly1.in_size
    out.out_size = butterfly2.out_size
    return out
