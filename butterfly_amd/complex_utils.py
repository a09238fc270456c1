"""Small complex-tensor helpers used by the modules (counterparts of the reference's
torch_butterfly/complex_utils.py; its cupy bridges have no use here: PyTorch multiplies complex
matrices on the device itself)."""
import math

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


Real2ComplexFn = _Real2Complex
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


IndexLastDim = _IndexLastDim
index_last_dim = _IndexLastDim.apply


def complex_mul(x, y):
    """Elementwise product (reference: torch_butterfly/complex_utils.py:complex_mul)."""
    return x * y


def complex_matmul(X, Y):
    """Batched matrix product of real or complex tensors.  The reference routes complex
    operands through cupy or four real products (torch_butterfly/complex_utils.py:41-95) because
    its PyTorch had no complex matmul on the device; here the library product does it."""
    return X @ Y


def complex_matmul_torch(X, Y):
    """The complex product spelled as four real products (torch_butterfly/complex_utils.py:41-44)."""
    return torch.complex(X.real @ Y.real - X.imag @ Y.imag, X.real @ Y.imag + X.imag @ Y.real)


class ComplexLinear(nn.Module):
    """``nn.Linear`` with complex64 weight (out_features, in_features) and bias
    (torch_butterfly/complex_utils.py:153-186).  Initialised as nn.Linear is, real and imaginary
    parts drawn alike and the weight divided by sqrt(2) so that its variance matches the real
    layer's (the reference means to do this; its ``reset_parameters`` names an undefined
    variable at that step and raises)."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.weight = nn.Parameter(torch.empty(out_features, in_features, dtype=torch.complex64))
        if bias:
            self.bias = nn.Parameter(torch.empty(out_features, dtype=torch.complex64))
        else:
            self.register_parameter('bias', None)
        self.reset_parameters()

    def reset_parameters(self) -> None:
        # nn.Linear's kaiming_uniform_(a=sqrt(5)) is uniform in +-1/sqrt(fan_in), for weight and bias alike
        bound = 1 / math.sqrt(self.in_features)
        with torch.no_grad():
            torch.view_as_real(self.weight).uniform_(-bound, bound)
            self.weight /= math.sqrt(2)
            if self.bias is not None:
                torch.view_as_real(self.bias).uniform_(-bound, bound)

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        output = complex_matmul(complex_reshape(input, -1, input.size(-1)), self.weight.t())
        output = output.reshape(*input.shape[:-1], output.shape[-1])
        return output if self.bias is None else output + self.bias

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}"
