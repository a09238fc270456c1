"""Learnable diagonal matrix (reference: torch_butterfly/diagonal.py)."""
import torch
from torch import nn

from .complex_utils import real_dtype_to_complex


class Diagonal(nn.Module):
    """output = input * diagonal, broadcast over leading dimensions."""

    def __init__(self, size=None, complex=False, diagonal_init=None):
        super().__init__()
        if diagonal_init is not None:
            self.diagonal = nn.Parameter(diagonal_init.detach().clone())
            self.complex = self.diagonal.is_complex()
        else:
            if size is None:
                raise ValueError("either size or diagonal_init is required")
            self.complex = complex
            dtype = torch.get_default_dtype()
            if complex:
                dtype = real_dtype_to_complex[dtype]
            self.diagonal = nn.Parameter(torch.randn(size, dtype=dtype))
        self.size = self.diagonal.shape[-1]
        self.diagonal._is_structured = True

    def forward(self, input):
        return input * self.diagonal
