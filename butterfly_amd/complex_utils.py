"""Small complex-tensor helpers used by the modules (counterparts of the pieces of the
reference's torch_butterfly/complex_utils.py:100-150 that sit on the multiply path)."""
import torch
from torch import nn

real_dtype_to_complex = {torch.float32: torch.complex64, torch.float64: torch.complex128}
complex_dtype_to_real = {v: k for k, v in real_dtype_to_complex.items()}


def complex_reshape(x, *shape):
    """Reshape that also works for non-contiguous complex tensors."""
    if not x.is_complex():
        return x.reshape(*shape)
    return torch.view_as_complex(torch.view_as_real(x).reshape(*shape, 2))


class _Real2Complex(torch.autograd.Function):
    """Cast real -> complex; the gradient is the real part of the incoming gradient."""

    @staticmethod
    def forward(ctx, x):
        return x.to(real_dtype_to_complex[x.dtype])

    @staticmethod
    def backward(ctx, grad):
        return grad.real


real2complex = _Real2Complex.apply


class Real2Complex(nn.Module):
    def forward(self, input):
        return real2complex(input)


class Complex2Real(nn.Module):
    def forward(self, input):
        return input.real


class _IndexLastDim(torch.autograd.Function):
    """Gather along the last dimension with a permutation; backward scatters."""

    @staticmethod
    def forward(ctx, x, permutation):
        ctx.save_for_backward(permutation)
        return x[..., permutation]

    @staticmethod
    def backward(ctx, grad):
        (permutation,) = ctx.saved_tensors
        out = torch.empty_like(grad)
        out[..., permutation] = grad
        return out, None


index_last_dim = _IndexLastDim.apply


def complex_mul(x, y):
    """Elementwise product (reference: torch_butterfly/complex_utils.py:complex_mul)."""
    return x * y


def complex_matmul(x, y):
    """Batched matrix product of real or complex tensors.  The reference routes complex
    operands through cupy or four real products (torch_butterfly/complex_utils.py:41-95) because
    its PyTorch had no complex matmul on the device; here the library product does it."""
    return x @ y
