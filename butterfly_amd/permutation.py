"""Fixed permutations on the multiply path: the FFT bit reversal and a module that applies a
stored permutation (reference: torch_butterfly/permutation.py:14-30,55-78)."""
import numpy as np
import torch
from torch import nn

from .complex_utils import index_last_dim


def bitreversal_permutation(n, pytorch_format=False):
    """perm[i] = i with its log2(n) bits reversed."""
    log_n = int(n).bit_length() - 1
    if n != 1 << log_n:
        raise ValueError("n must be a power of 2")
    idx = np.arange(n)
    perm = np.zeros(n, dtype=np.int64)
    for bit in range(log_n):
        perm |= ((idx >> bit) & 1) << (log_n - 1 - bit)
    return torch.from_numpy(perm) if pytorch_format else perm


def invert(perm):
    """Inverse permutation (numpy array or tensor)."""
    if isinstance(perm, torch.Tensor):
        inv = torch.empty_like(perm)
        inv[perm] = torch.arange(perm.numel(), dtype=perm.dtype, device=perm.device)
        return inv
    inv = np.empty_like(perm)
    inv[perm] = np.arange(perm.size)
    return inv


class FixedPermutation(nn.Module):
    """output[..., i] = input[..., permutation[i]]."""

    def __init__(self, permutation: torch.Tensor) -> None:
        super().__init__()
        self.register_buffer("permutation", permutation)

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        return index_last_dim(input, self.permutation)
