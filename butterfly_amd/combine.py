"""Twiddle algebra: fold a diagonal into a Butterfly, concatenate two Butterflies, tensor and
Kronecker products, change of stride direction (reference: torch_butterfly/combine.py)."""
import copy

import torch
from torch import nn
from torch.nn import functional as F

from .butterfly import Butterfly
from .permutation import FixedPermutation, FusedSequential, bitreversal_permutation


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


class TensorProduct(nn.Module):
    """map1 along the last dimension, then map2 along the one before it: (*, n2, n1) -> (*, m2, m1)
    (reference: torch_butterfly/combine.py:80-98)."""

    def __init__(self, map1, map2) -> None:
        super().__init__()
        self.map1 = map1
        self.map2 = map2

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        rows_done = self.map1(input)
        return self.map2(rows_done.transpose(-1, -2)).transpose(-1, -2)


def butterfly_kronecker(butterfly1: Butterfly, butterfly2: Butterfly) -> Butterfly:
    """The Butterfly of size n1 * n2 equal to butterfly2 (x) butterfly1 on inputs flattened
    from (n2, n1): element index = i2 * n1 + i1, so butterfly1 owns the low log2(n1) index bits
    and butterfly2 the high ones.  A stage of butterfly1 then sees every pair index modulo
    n1 / 2 (its factors tiled n2 times), a stage of butterfly2 sees the pair index divided by n1
    (each factor repeated n1 times); with increasing stride butterfly1's stages come first.
    Both must have the same stride direction, one stack, one block and no bias
    (reference: torch_butterfly/combine.py:101-130)."""
    if butterfly1.increasing_stride != butterfly2.increasing_stride:
        raise ValueError("the factors must have the same stride direction")
    if butterfly1.complex != butterfly2.complex:
        raise ValueError("the factors must both be real or both be complex")
    for b in (butterfly1, butterfly2):
        if b.bias is not None or b.nstacks != 1 or b.nblocks != 1:
            raise ValueError("butterfly_kronecker needs nstacks == 1, nblocks == 1 and no bias")
    n1, n2 = 1 << butterfly1.log_n, 1 << butterfly2.log_n
    low = butterfly1.twiddle.detach().repeat(1, 1, 1, n2, 1, 1)
    high = butterfly2.twiddle.detach().repeat_interleave(n1, dim=3)
    stages = (low, high) if butterfly1.increasing_stride else (high, low)
    out = Butterfly(n1 * n2, n1 * n2, bias=False, complex=butterfly1.complex,
                    increasing_stride=butterfly1.increasing_stride, init=torch.cat(stages, dim=2))
    out.in_size = butterfly1.in_size * butterfly2.in_size
    out.out_size = butterfly1.out_size * butterfly2.out_size
    return out


def permutation_kronecker(perm1: FixedPermutation, perm2: FixedPermutation) -> FixedPermutation:
    """The permutation of n1 * n2 flattened (n2, n1) elements that applies perm1 within rows and
    perm2 across rows (reference: torch_butterfly/combine.py:133-139)."""
    p1, p2 = perm1.permutation, perm2.permutation
    n1 = p1.shape[-1]
    return FixedPermutation((p2.unsqueeze(1) * n1 + p1.unsqueeze(0)).reshape(-1))


def flip_increasing_stride(butterfly: Butterfly) -> nn.Module:
    """The same matrix with the opposite stride direction, between two bit reversals.

    Conjugating with the bit reversal P of the element index sends the stage pairing bit l to
    one pairing bit log_n - 1 - l and keeps its position in the block; the pair index of a
    stage is the element index with the paired bit removed, so it gets bit-reversed as a
    (log_n - 1)-bit number.  Hence B = P B' P with B'.twiddle[..., i] = B.twiddle[..., br(i)]
    (reference: torch_butterfly/combine.py:142-160)."""
    n = 1 << butterfly.log_n
    if butterfly.bias is not None or butterfly.in_size != n or butterfly.out_size != n:
        raise ValueError("flip_increasing_stride needs a square power-of-2 Butterfly without bias")
    flipped = copy.deepcopy(butterfly)
    flipped.increasing_stride = not butterfly.increasing_stride
    if n > 2:
        pairs = bitreversal_permutation(n // 2, pytorch_format=True).to(butterfly.twiddle.device)
        with torch.no_grad():
            flipped.twiddle.copy_(butterfly.twiddle.detach()[:, :, :, pairs])
    br = bitreversal_permutation(n, pytorch_format=True).to(butterfly.twiddle.device)
    return FusedSequential(FixedPermutation(br), flipped, FixedPermutation(br.clone()))
