"""``Butterfly``: an ``nn.Linear``-compatible layer whose weight is a product of butterfly
factors, evaluated by the native multiply.

Mirrors the constructor, parameters (``twiddle``, ``bias``), state-dict layout and forward
flags of the reference module (torch_butterfly/butterfly.py:15-207).
"""
import math
import numbers

import torch
from torch import nn

from .complex_utils import complex_reshape, real_dtype_to_complex
from .multiply import butterfly_multiply, butterfly_multiply_bias, butterfly_multiply_perm

_INITS = ("empty", "randn", "ortho", "identity", "fft_no_br", "ifft_no_br")


def _ortho_real(core_shape):
    """Random 2x2 rotations / reflections [[d c, -d s], [s, c]], d = +-1."""
    theta = torch.rand(core_shape) * (2 * math.pi)
    c, s = theta.cos(), theta.sin()
    d = torch.randint(0, 2, core_shape, dtype=c.dtype) * 2 - 1
    return torch.stack((torch.stack((d * c, -d * s), -1), torch.stack((s, c), -1)), -2)


def _ortho_complex(core_shape):
    """Haar-distributed U(2) factors: [[e^{i(a+p)} c, e^{i(a+x)} s], [-e^{i(a-x)} s, e^{i(a-p)} c]]."""
    phi = torch.rand(core_shape).sqrt().asin()
    c, s = phi.cos(), phi.sin()
    alpha, psi, chi = torch.rand((3,) + tuple(core_shape)) * (2 * math.pi)
    top = torch.stack((torch.exp(1j * (alpha + psi)) * c, torch.exp(1j * (alpha + chi)) * s), -1)
    bot = torch.stack((-torch.exp(1j * (alpha - chi)) * s, torch.exp(1j * (alpha - psi)) * c), -1)
    return torch.stack((top, bot), -2)


def scale_twiddle(twiddle, increasing_stride, in_scale=None, out_scale=None):
    """twiddle (stacks, nblocks, log_n, n/2, 2, 2) of the product B with diag(out_scale) B
    diag(in_scale) folded in: the columns of the first applied factor take in_scale, the rows
    of the last applied one out_scale.  in_scale has up to n entries (every stack reads the same
    input), out_scale up to stacks * n (the stacks' outputs side by side); missing entries are 1.
    Differentiable in all three arguments."""
    for v in (in_scale, out_scale):
        if v is not None and v.is_complex() and not twiddle.is_complex():
            raise ValueError("a complex diagonal cannot be folded into real factors")
    if twiddle.is_cuda and twiddle.dtype in (torch.float32, torch.complex64):
        # one small kernel forward, two backward (n-sized work, a single autograd node)
        cast = lambda v: None if v is None else v.to(twiddle.dtype)
        return torch.ops.torch_butterfly.butterfly_scale_twiddle(twiddle, cast(in_scale), cast(out_scale),
                                                                 increasing_stride)
    stacks, nblocks, log_n, half = twiddle.shape[:4]
    n = 1 << log_n

    def pairs(vec, rows, stride):
        # (rows, n) entries by element -> (rows, n/2, 2) by pair index and position in the pair
        if vec.shape[-1] < rows * n:
            vec = torch.nn.functional.pad(vec, (0, rows * n - vec.shape[-1]), value=1.0)
        return vec.reshape(rows, n // (2 * stride), 2, stride).transpose(-1, -2).reshape(rows, half, 2)

    flat = twiddle.reshape(stacks, nblocks * log_n, half, 2, 2)
    first, last = flat[:, 0], flat[:, -1]
    if in_scale is not None:
        stride = 1 if increasing_stride else half
        cols = pairs(in_scale, 1, stride)[:, :, None, :]
        if nblocks * log_n == 1:
            last = last * cols
        first = first * cols
    if out_scale is not None:
        last_increasing = increasing_stride != ((nblocks - 1) % 2 == 1)
        stride = half if last_increasing else 1
        last = last * pairs(out_scale, stacks, stride)[:, :, :, None]
        if nblocks * log_n == 1:
            first = last
    if nblocks * log_n == 1:
        return last.reshape(twiddle.shape)
    return torch.cat((first.unsqueeze(1), flat[:, 1:-1], last.unsqueeze(1)), 1).reshape(twiddle.shape)


class Butterfly(nn.Module):
    """Product of ``nblocks * log_n`` butterfly factors (block-diagonal 2x2 stages).

    Parameters:
        in_size, out_size: like ``nn.Linear``.  ``n`` is ``in_size`` rounded up to a power of 2
            and ``nstacks = ceil(out_size / n)`` independent products are stacked.
        bias: learn an additive bias of size ``out_size``.
        complex: complex64/128 twiddle instead of real.
        increasing_stride: the first block multiplies with stride 1, 2, ..., n/2 (else
            n/2, ..., 1); the direction alternates from block to block.
        init: a tensor of shape (nstacks, nblocks, log_n, n/2, 2, 2), or one of 'randn',
            'ortho', 'identity', 'fft_no_br', 'ifft_no_br', 'empty'.
        nblocks: number of alternating B / B^T blocks.
    """

    def __init__(self, in_size, out_size, bias=True, complex=False, increasing_stride=True,
                 init="randn", nblocks=1):
        super().__init__()
        if nblocks < 1:
            raise ValueError("nblocks must be >= 1")
        self.in_size = in_size
        self.out_size = out_size
        self.log_n = int(math.ceil(math.log2(in_size)))
        self.n = 1 << self.log_n
        self.nstacks = -(-out_size // self.n)
        self.complex = complex
        self.increasing_stride = increasing_stride
        self.nblocks = nblocks
        dtype = torch.get_default_dtype()
        if complex:
            dtype = real_dtype_to_complex[dtype]
        shape = (self.nstacks, nblocks, self.log_n, self.n // 2, 2, 2)
        if isinstance(init, torch.Tensor):
            if tuple(init.shape) != shape or init.dtype != dtype:
                raise ValueError(f"init tensor must have shape {shape} and dtype {dtype}")
            self.init = None
            self.twiddle = nn.Parameter(init.clone())
        else:
            if init not in _INITS:
                raise ValueError(f"init must be a tensor or one of {_INITS}")
            self.init = init
            self.twiddle = nn.Parameter(torch.empty(shape, dtype=dtype))
        if bias:
            self.bias = nn.Parameter(torch.empty(out_size, dtype=dtype))
        else:
            self.register_parameter("bias", None)
        self.twiddle._is_structured = True  # lets optimisers exempt it from weight decay
        self.reset_parameters()

    def reset_parameters(self):
        if self.bias is not None:
            bound = 1 / math.sqrt(self.in_size)  # same rule as nn.Linear
            nn.init.uniform_(self.bias, -bound, bound)
        tw = self.twiddle
        if self.init in (None, "empty"):
            return
        with torch.no_grad():
            if self.init == "randn":
                # variance 1/2 per entry keeps the output variance equal to the input's
                tw.copy_(torch.randn(tw.shape, dtype=tw.dtype) / math.sqrt(2))
            elif self.init == "ortho":
                core = tw.shape[:-2]
                tw.copy_(_ortho_complex(core) if self.complex else _ortho_real(core))
            elif self.init == "identity":
                tw.copy_(torch.eye(2, dtype=tw.dtype).expand(tw.shape))
            else:
                if not self.complex:
                    raise ValueError("fft_no_br / ifft_no_br init needs complex=True")
                from . import special
                make = special.fft if self.init == "fft_no_br" else special.ifft
                b = make(self.n, normalized=True, br_first=self.increasing_stride, with_br_perm=False)
                tw[:, 0] = b.twiddle
                if self.nblocks > 1:
                    tw[:, 1:] = torch.eye(2, dtype=tw.dtype)

    def forward(self, input, transpose=False, conjugate=False, subtwiddle=False, in_perm=None, out_index=None,
                in_scale=None, out_scale=None):
        """input (batch, *, in_size) -> (batch, *, out_size).

        transpose / conjugate apply the transposed / conjugated matrix; subtwiddle uses only
        the leading part of the parameters for a shorter input (output is then
        nstacks * n' wide, n' the input size rounded up to a power of 2).

        in_perm / out_index (int32 tables of n entries, see FixedPermutation.column_table): a
        fixed permutation in front of / behind the layer, applied by the layer's own kernels;
        they describe the untransposed layer (transpose swaps their roles).

        in_scale / out_scale (vectors of in_size / out_size entries): a diagonal matrix directly
        in front of / behind the layer (between the layer and the permutation of in_perm /
        out_index, if there is one).  They are multiplied into the first / last factor, an
        n-sized operation that autograd differentiates, instead of into the activations."""
        if in_scale is not None or out_scale is not None:
            if subtwiddle or transpose:
                raise ValueError("in_scale / out_scale cannot be combined with subtwiddle or transpose")
            if out_scale is not None and self.bias is not None:
                raise ValueError("a diagonal behind the layer cannot be folded past the bias")
        if in_perm is not None or out_index is not None:
            if subtwiddle:
                raise ValueError("column tables cannot be combined with subtwiddle")
            if out_index is not None and self.nstacks != 1:
                raise ValueError("a permutation behind the layer needs nstacks == 1")
            if transpose:
                in_perm, out_index = out_index, in_perm
        twiddle = self.effective_twiddle()
        x = self.pre_process(input)
        output_size = self.out_size if self.nstacks == 1 else None
        if subtwiddle:
            log_n = int(math.ceil(math.log2(input.size(-1))))
            half = (1 << log_n) // 2
            if self.increasing_stride:
                twiddle = twiddle[:, :, :log_n, :half]
            else:
                twiddle = twiddle[:, :, self.log_n - log_n:, :half]
            output_size = None
        if conjugate and self.complex:
            twiddle = twiddle.conj()
        if in_scale is not None or out_scale is not None:
            twiddle = scale_twiddle(twiddle, self.increasing_stride, in_scale, out_scale)
        if transpose:
            # (prod of stages)^T: transpose every 2x2 and reverse the stage and block order
            twiddle = twiddle.transpose(-1, -2).flip([1, 2])
            last_inc = self.increasing_stride != ((self.nblocks - 1) % 2 == 1)
            inc = not last_inc
        else:
            inc = self.increasing_stride
        if in_perm is not None or out_index is not None:
            cols = output_size if output_size is not None else 1 << twiddle.shape[2]
            bias = None if self.bias is None else self.bias_rows(cols, subtwiddle)
            x = butterfly_multiply_perm(twiddle, x, in_perm, out_index, bias, inc, output_size)
        elif self.bias is None:
            x = butterfly_multiply(twiddle, x, inc, output_size)
        else:
            # the kernel that writes the output adds the bias, laid out as (stacks, columns)
            cols = output_size if output_size is not None else 1 << twiddle.shape[2]
            x = butterfly_multiply_bias(twiddle, x, self.bias_rows(cols, subtwiddle), inc, output_size)
        return self.post_process(input, x, out_size=x.size(-1) if subtwiddle else None, add_bias=False)

    def effective_twiddle(self):
        """(stacks, nblocks, log_n, n/2, 2, 2) factors the multiply runs with."""
        return self.twiddle

    def bias_rows(self, cols, subtwiddle=False):
        """The bias as the (stacks, cols) tensor that lines up with the multiply's output:
        post_process keeps the first out_size columns of the flattened stacks (with subtwiddle,
        the columns of one stack); the rest is padding."""
        total = self.nstacks * cols
        kept = cols if subtwiddle else self.out_size
        bias = self.bias[:kept]
        if bias.shape[0] != kept:
            raise ValueError("bias is shorter than the output")
        if kept < total:
            bias = torch.nn.functional.pad(bias, (0, total - kept))
        return bias.reshape(self.nstacks, cols)

    def pre_process(self, input):
        size = input.size(-1)
        x = complex_reshape(input, -1, size)
        return x.unsqueeze(1).expand(x.shape[0], self.nstacks, size)

    def post_process(self, input, output, out_size=None, add_bias=True):
        out_size = self.out_size if out_size is None else out_size
        batch = output.shape[0]
        flat = output.reshape(batch, self.nstacks * output.size(-1))
        if flat.shape[-1] != out_size:
            flat = flat[:, :out_size]
        if self.bias is not None and add_bias:
            flat = flat + self.bias[:out_size]
        return flat.reshape(*input.shape[:-1], out_size)

    def __imul__(self, scale):
        """Scale the whole matrix by a non-negative number, spread evenly over the stages."""
        if not isinstance(scale, numbers.Number) or scale < 0:
            raise ValueError("scale must be a non-negative number")
        self.twiddle *= scale ** (1.0 / (self.twiddle.shape[1] * self.twiddle.shape[2]))
        return self

    def diagonal_multiply_(self, diagonal, diag_first):
        from .combine import diagonal_butterfly
        return diagonal_butterfly(self, diagonal, diag_first, inplace=True)

    def to_base4(self):
        from .butterfly_base4 import ButterflyBase4
        from .multiply_base4 import twiddle_base2_to_base4
        with torch.no_grad():
            tw4, tw2 = twiddle_base2_to_base4(self.twiddle, self.increasing_stride)
        new = ButterflyBase4(self.in_size, self.out_size, self.bias is not None, self.complex,
                             self.increasing_stride, init=(tw4, tw2),
                             nblocks=self.nblocks).to(self.twiddle.device)
        if new.bias is not None:
            with torch.no_grad():
                new.bias.copy_(self.bias)
        return new

    def extra_repr(self):
        return (f"in_size={self.in_size}, out_size={self.out_size}, bias={self.bias is not None}, "
                f"complex={self.complex}, increasing_stride={self.increasing_stride}, "
                f"init={self.init}, nblocks={self.nblocks}")


class ButterflyUnitary(Butterfly):
    """Butterfly layer constrained to be unitary: every 2x2 factor is a U(2) element
    [[e^{i(a+p)} cos f, e^{i(a+x)} sin f], [-e^{i(a-x)} sin f, e^{i(a-p)} cos f]] built from the
    four real angles (f, a, p, x) stored in ``twiddle[..., 4]``.  Complex; same forward flags as
    ``Butterfly`` (reference: torch_butterfly/butterfly.py:210-305)."""

    def __init__(self, in_size, out_size, bias=True, increasing_stride=True, nblocks=1):
        nn.Module.__init__(self)
        if nblocks < 1:
            raise ValueError("nblocks must be >= 1")
        self.in_size = in_size
        self.out_size = out_size
        self.log_n = int(math.ceil(math.log2(in_size)))
        self.n = 1 << self.log_n
        self.nstacks = -(-out_size // self.n)
        self.complex = True
        self.increasing_stride = increasing_stride
        self.nblocks = nblocks
        self.init = "ortho"
        self.twiddle = nn.Parameter(torch.empty(self.nstacks, nblocks, self.log_n, self.n // 2, 4))
        if bias:
            self.bias = nn.Parameter(torch.empty(out_size, dtype=real_dtype_to_complex[torch.get_default_dtype()]))
        else:
            self.register_parameter("bias", None)
        self.twiddle._is_structured = True
        self.reset_parameters()

    def reset_parameters(self):
        # Haar measure on U(2): sin^2(f) uniform, the three phases uniform
        core = self.twiddle.shape[:-1]
        phi = torch.rand(core).sqrt().asin()
        phases = torch.rand((3,) + tuple(core)) * (2 * math.pi)
        with torch.no_grad():
            self.twiddle.copy_(torch.stack((phi, phases[0], phases[1], phases[2]), -1))
        if self.bias is not None:
            bound = 1 / math.sqrt(self.in_size)
            nn.init.uniform_(self.bias, -bound, bound)

    def effective_twiddle(self):
        phi, alpha, psi, chi = self.twiddle.unbind(-1)
        c, s = phi.cos(), phi.sin()

        def polar(r, angle):
            return torch.complex(r * angle.cos(), r * angle.sin())

        top = torch.stack((polar(c, alpha + psi), polar(s, alpha + chi)), -1)
        bot = torch.stack((polar(-s, alpha - chi), polar(c, alpha - psi)), -1)
        return torch.stack((top, bot), -2)

    __imul__ = None
    to_base4 = None
    diagonal_multiply_ = None

    def extra_repr(self):
        return (f"in_size={self.in_size}, out_size={self.out_size}, bias={self.bias is not None}, "
                f"increasing_stride={self.increasing_stride}, nblocks={self.nblocks}")


class ButterflyBmm(Butterfly):
    """``matrix_batch`` independent Butterfly layers applied to the matching slices of the
    input: (batch, *, matrix_batch, in_size) -> (batch, *, matrix_batch, out_size).  The
    matrices ride on the stack dimension of one multiply (reference:
    torch_butterfly/butterfly.py:308-397)."""

    def __init__(self, in_size, out_size, matrix_batch=1, bias=True, complex=False, increasing_stride=True,
                 init="randn", nblocks=1):
        nn.Module.__init__(self)
        if nblocks < 1:
            raise ValueError("nblocks must be >= 1")
        self.in_size = in_size
        self.out_size = out_size
        self.matrix_batch = matrix_batch
        self.log_n = int(math.ceil(math.log2(in_size)))
        self.n = 1 << self.log_n
        self.nstacks = -(-out_size // self.n)
        self.complex = complex
        self.increasing_stride = increasing_stride
        self.nblocks = nblocks
        dtype = torch.get_default_dtype()
        if complex:
            dtype = real_dtype_to_complex[dtype]
        shape = (matrix_batch * self.nstacks, nblocks, self.log_n, self.n // 2, 2, 2)
        if isinstance(init, torch.Tensor):
            if tuple(init.shape) != shape or init.dtype != dtype:
                raise ValueError(f"init tensor must have shape {shape} and dtype {dtype}")
            self.init = None
            self.twiddle = nn.Parameter(init.clone())
        else:
            if init not in _INITS:
                raise ValueError(f"init must be a tensor or one of {_INITS}")
            self.init = init
            self.twiddle = nn.Parameter(torch.empty(shape, dtype=dtype))
        if bias:
            self.bias = nn.Parameter(torch.empty(matrix_batch, out_size, dtype=dtype))
        else:
            self.register_parameter("bias", None)
        self.twiddle._is_structured = True
        self.reset_parameters()

    def forward(self, input, transpose=False, conjugate=False):
        return super().forward(input, transpose, conjugate, subtwiddle=False)

    def bias_rows(self, cols, subtwiddle=False):
        total = self.nstacks * cols
        bias = self.bias[:, :self.out_size]
        if self.out_size < total:
            bias = torch.nn.functional.pad(bias, (0, total - self.out_size))
        return bias.reshape(self.matrix_batch * self.nstacks, cols)

    def pre_process(self, input):
        size = input.size(-1)
        if input.size(-2) != self.matrix_batch:
            raise ValueError("the second to last dimension of the input must be matrix_batch")
        x = complex_reshape(input, -1, self.matrix_batch, size)
        x = x.unsqueeze(2).expand(x.shape[0], self.matrix_batch, self.nstacks, size)
        return x.reshape(x.shape[0], self.matrix_batch * self.nstacks, size)

    def post_process(self, input, output, out_size=None, add_bias=True):
        out_size = self.out_size if out_size is None else out_size
        batch = output.shape[0]
        flat = output.reshape(batch, self.matrix_batch, self.nstacks * output.size(-1))
        if flat.shape[-1] != out_size:
            flat = flat[:, :, :out_size]
        if self.bias is not None and add_bias:
            flat = flat + self.bias[:, :out_size]
        return flat.reshape(*input.shape[:-2], self.matrix_batch, out_size)

    to_base4 = None

    def extra_repr(self):
        return (f"in_size={self.in_size}, out_size={self.out_size}, matrix_batch={self.matrix_batch}, "
                f"bias={self.bias is not None}, complex={self.complex}, "
                f"increasing_stride={self.increasing_stride}, init={self.init}, nblocks={self.nblocks}")
