"""The legacy ``butterfly`` package's layer and multiply functions on the native multiply.

Counterpart of the reference's butterfly/butterfly.py (``Butterfly``, ``ButterflyBmm``) and of
the functions it imports from butterfly/butterfly_multiply.py and butterfly/utils.py, with the
same names, argument order, parameter names and shapes, so code written against that package
(and its checkpoints) runs unchanged -- without apex and without the two compiled extensions
behind it.  Every function rewrites its parameters into the (nstack, nblocks, log n, n / 2, 2,
2) twiddle of ``butterfly_multiply`` with differentiable tensor operations (index gathers,
cos / sin, scaling by a diagonal) and makes ONE call to the native operator; autograd carries
the gradients back into the legacy layouts.

Legacy conventions handled here:
* complex numbers are real tensors with a trailing dimension of 2;
* ``twiddle[:, log_stride]`` belongs to that stride whatever the multiplication order;
* tied weights: (nstack, n - 1, 2, 2), entries stride - 1 .. 2 stride - 2 shared by all groups;
* orthogonal parameterisation: angles, factor [[cos, -sin], [sin, cos]];
* B B^T products: per block, log n factors with decreasing then log n with increasing stride;
* ODO: an orthogonal B B^T block with a diagonal in the middle;
* fast format: (nstack, stages, 2, n), stages in order of application, plane 0 the diagonal
  entry and plane 1 the off-diagonal entry of each element's output row (butterfly/utils.py:24-45).
"""
import math

import torch
import torch.nn.functional as F
from torch import nn

from .multiply import butterfly_multiply

_index_cache = {}


def _cached(key, device, make):
    entry = _index_cache.get((key, device))
    if entry is None:
        entry = make().to(device)
        _index_cache[(key, device)] = entry
    return entry


def _log2(n):
    m = int(n).bit_length() - 1
    if n != 1 << m:
        raise ValueError("size must be a power of 2")
    return m


def _pair_positions(m, log_stride):
    """Low element of every pair of the factor with this stride: pair i = h * stride + l sits
    at h * 2 stride + l."""
    i = torch.arange(1 << (m - 1))
    low = i & ((1 << log_stride) - 1)
    return ((i - low) << 1) + low


def _tied_index(m, device):
    """(log n, n / 2): entry of a tied twiddle that pair i of the stride-2^k factor uses."""
    def make():
        i = torch.arange(1 << (m - 1))
        return torch.stack([(1 << k) - 1 + (i & ((1 << k) - 1)) for k in range(m)])
    return _cached(("tied", m), device, make)


def _fast_gather_index(m, log_strides, device):
    """For stages with the given strides (in order of application): index into the flattened
    (2, n) fast slice of the four entries of every pair, shape (stages, n / 2 * 4)."""
    def make():
        n = 1 << m
        rows = []
        for k in log_strides:
            pos = _pair_positions(m, k)                                   # (n/2,)
            e = torch.stack((pos, pos + (1 << k)), -1)                    # element of output row r
            r = torch.arange(2).reshape(1, 2, 1)
            c = torch.arange(2).reshape(1, 1, 2)
            rows.append(((r ^ c) * n + e.unsqueeze(-1)).reshape(-1))     # plane (r != c), position e_r
        return torch.stack(rows)
    return _cached(("fast", m, tuple(log_strides)), device, make)


def _fast_scatter_index(m, device):
    """Inverse direction for strides 1, 2, ..., n / 2: index into a flattened (n / 2, 2, 2)
    factor of the entry that goes to [plane][element], shape (log n, 2 * n)."""
    def make():
        n = 1 << m
        e = torch.arange(n)
        rows = []
        for k in range(m):
            r = (e >> k) & 1
            pair = ((e >> (k + 1)) << k) | (e & ((1 << k) - 1))
            diag = pair * 4 + r * 3                                       # T[r][r]
            off = pair * 4 + r * 2 + (1 - r)                              # T[r][1 - r]
            rows.append(torch.cat((diag, off)))
        return torch.stack(rows)
    return _cached(("unfast", m), device, make)


def twiddle_normal_to_fast_format(twiddle):
    """(nstack, log n, n / 2, 2, 2) -> (nstack, log n, 2, n) (butterfly/utils.py:24-45)."""
    nstack, m, half = twiddle.shape[:3]
    n = 2 * half
    idx = _fast_scatter_index(m, twiddle.device).unsqueeze(0).expand(nstack, m, 2 * n)
    return twiddle.reshape(nstack, m, 2 * n).gather(2, idx).reshape(nstack, m, 2, n)


def _fast_to_stages(twiddle_fast, m, log_strides):
    """Fast slices (nstack, stages, 2, n) whose j-th slice has stride 2^log_strides[j] ->
    (nstack, stages, n / 2, 2, 2)."""
    nstack, stages = twiddle_fast.shape[:2]
    n = 1 << m
    idx = _fast_gather_index(m, log_strides, twiddle_fast.device).unsqueeze(0).expand(nstack, stages, 2 * n)
    return twiddle_fast.reshape(nstack, stages, 2 * n).gather(2, idx).reshape(nstack, stages, n // 2, 2, 2)


def _rotation(theta):
    c, s = torch.cos(theta), torch.sin(theta)
    return torch.stack((torch.stack((c, -s), -1), torch.stack((s, c), -1)), -2)


def _as_complex(t):
    try:
        return torch.view_as_complex(t)
    except RuntimeError:
        return torch.view_as_complex(t.contiguous())


# ---- helpers of butterfly/complex_utils.py and butterfly/utils.py on (..., 2) real pairs ------------

def real_to_complex(X):
    """(...) -> (..., 2) with zero imaginary parts (butterfly/complex_utils.py:40-47)."""
    return torch.stack((X, torch.zeros_like(X)), dim=-1)


def conjugate(X):
    """(butterfly/complex_utils.py:50-75)"""
    return torch.view_as_real(_as_complex(X).conj().resolve_conj())


def complex_mul(X, Y):
    """Elementwise product with broadcasting (butterfly/complex_utils.py:78-131)."""
    shape = torch.broadcast_shapes(X.shape, Y.shape)
    return torch.view_as_real(_as_complex(X.expand(shape)) * _as_complex(Y.expand(shape)))


def complex_matmul(X, Y):
    """(..., n, m, 2) x (..., m, p, 2) -> (..., n, p, 2) (butterfly/complex_utils.py:162-201)."""
    return torch.view_as_real(_as_complex(X) @ _as_complex(Y))


conjugate_torch = conjugate
complex_mul_torch = complex_mul
complex_matmul_torch = complex_matmul


def bitreversal_permutation(n):
    """numpy array: perm[i] = i with its log2(n) bits reversed (butterfly/utils.py:8-21)."""
    from .permutation import bitreversal_permutation as table
    return table(n)


def _multiply(twiddle, input, increasing_stride):
    """twiddle (nstack, nblocks, log n, n / 2, 2, 2) in order of application (pairs of reals
    appended for complex), input (batch, nstack, n[, 2])."""
    if input.dim() == 4:
        out = butterfly_multiply(_as_complex(twiddle), _as_complex(input), increasing_stride)
        return torch.view_as_real(out)
    return butterfly_multiply(twiddle, input, increasing_stride)


def _alternating_strides(m, nchunks):
    """Strides of B B^T products in order of application: decreasing in even slices of log n
    factors, increasing in odd ones."""
    out = []
    for k in range(nchunks):
        out += list(range(m)) if k % 2 == 1 else list(range(m - 1, -1, -1))
    return out


# ---- functions of butterfly/butterfly_multiply.py ---------------------------------------------------

def butterfly_mult_untied(twiddle, input, increasing_stride=True, is_training=True, fast=False):
    """twiddle (nstack, log n, n / 2, 2, 2[, 2]) indexed by log_stride, or with ``fast`` the
    fast format (nstack, log n, 2, n) in order of application (real only);
    input (batch, nstack, n[, 2]) (butterfly_multiply.py:126-219)."""
    m = _log2(input.shape[2])
    if fast:
        if input.dim() == 4:
            raise ValueError("the fast format is defined for real twiddles only")
        strides = list(range(m)) if increasing_stride else list(range(m - 1, -1, -1))
        stages = _fast_to_stages(twiddle, m, strides)
    else:
        stages = twiddle if increasing_stride else twiddle.flip(1)
    return _multiply(stages.unsqueeze(1), input, increasing_stride)


def butterfly_mult(twiddle, input, increasing_stride=True):
    """Tied weights: twiddle (nstack, n - 1, 2, 2[, 2]) (butterfly_multiply.py:43-123)."""
    m = _log2(input.shape[2])
    return butterfly_mult_untied(twiddle[:, _tied_index(m, twiddle.device)], input, increasing_stride)


def butterfly_ortho_mult_tied(twiddle, input, increasing_stride):
    """Angles (nstack, n - 1) (butterfly_multiply.py:222-269)."""
    return butterfly_mult(_rotation(twiddle), input, increasing_stride)


def butterfly_ortho_mult_untied(twiddle, input, increasing_stride):
    """Angles (nstack, log n, n / 2) (butterfly_multiply.py:272-319)."""
    return butterfly_mult_untied(_rotation(twiddle), input, increasing_stride)


def bbt_mult_untied(twiddle, input, fast=True):
    """twiddle (nstack, nblocks * 2 log n, n / 2, 2, 2): per block the first log n factors,
    flipped, run with decreasing stride and the rest with increasing stride -- so the factors
    apply in storage order (butterfly_multiply.py:359-386).  With ``fast`` the twiddle is
    (nstack, nblocks * 2 log n, 2, n), likewise in order of application."""
    m = _log2(input.shape[2])
    nchunks = twiddle.shape[1] // m
    if nchunks * m != twiddle.shape[1] or nchunks % 2:
        raise ValueError("twiddle must hold nblocks * 2 * log n factors")
    if fast and twiddle.dim() == 4:
        twiddle = _fast_to_stages(twiddle, m, _alternating_strides(m, nchunks))
    nstack = twiddle.shape[0]
    return _multiply(twiddle.reshape(nstack, nchunks, m, *twiddle.shape[2:]), input, False)


def bbt_ortho_mult_untied(twiddle, input):
    """Angles (nstack, nblocks * 2 log n, n / 2) (butterfly_multiply.py:431-449)."""
    return bbt_mult_untied(_rotation(twiddle), input, fast=False)


def _conv2d_patches(twiddle, input, kernel_size, padding):
    """The (batch * h_out * w_out, kernel_size^2 * c_out / c_in, c_in) operand of the
    convolution-as-butterflies: one row per output pixel, one stack per kernel position (and
    copy of the input channels, when c_out is a multiple of c_in)
    (butterfly_multiply.py:509-520)."""
    b_in, c_in, h_in, w_in = input.shape
    positions = kernel_size * kernel_size
    if twiddle.shape[0] % positions:
        raise ValueError("twiddle must hold a multiple of kernel_size^2 stacks")
    copies = twiddle.shape[0] // positions
    if c_in != 1 << _log2(c_in):
        raise ValueError("c_in must be a power of 2")
    h_out = h_in + 2 * padding - (kernel_size - 1)
    w_out = w_in + 2 * padding - (kernel_size - 1)
    patches = F.unfold(input, kernel_size=kernel_size, dilation=1, padding=padding, stride=1)
    patches = patches.view(b_in, c_in, positions, h_out * w_out).permute(0, 3, 2, 1)
    patches = patches.reshape(b_in * h_out * w_out, positions, 1, c_in)
    return patches.expand(-1, positions, copies, c_in).reshape(b_in * h_out * w_out, positions * copies, c_in)


def butterfly_mult_conv2d(twiddle, input, kernel_size, padding, increasing_stride=True):
    """twiddle (nstack, log n, n / 2, 2, 2), n = c_in, nstack = kernel_size^2 * c_out / c_in;
    input (batch, c_in, h, w) -> (batch * h_out * w_out, nstack, c_in): every kernel position's
    patch through its own butterflies, stride 1, square kernels (butterfly_multiply.py:491-583)."""
    return butterfly_mult_untied(twiddle, _conv2d_patches(twiddle, input, kernel_size, padding), increasing_stride)


def bbt_mult_conv2d(twiddle, input, kernel_size, padding):
    """The same with B B^T products: twiddle (nstack, nblocks * 2 log n, n / 2, 2, 2)
    (butterfly_multiply.py:626-664)."""
    return bbt_mult_untied(twiddle, _conv2d_patches(twiddle, input, kernel_size, padding), fast=False)


def butterfly_mult_factors(twiddle, input, increasing_stride=True, return_intermediates=False):
    """Tied weights without a stack dimension: twiddle (n - 1, 2, 2[, 2]), input (batch, n[, 2])
    (butterfly_multiply.py:696-730).  The reference runs one kernel per factor, for debugging;
    here the product is one call, and only ``return_intermediates`` (the input and the value
    after every factor, stacked) walks the factors one by one, in PyTorch operations."""
    if not return_intermediates:
        return butterfly_mult(twiddle.unsqueeze(0), input.unsqueeze(1), increasing_stride).squeeze(1)
    cplx = input.dim() == 3
    n = input.shape[1]
    m = _log2(n)
    x = _as_complex(input) if cplx else input
    t = _as_complex(twiddle) if cplx else twiddle
    values = [x]
    for log_stride in (range(m) if increasing_stride else range(m - 1, -1, -1)):
        stride = 1 << log_stride
        f = t[stride - 1:2 * stride - 1]                             # (stride, 2, 2)
        pairs = values[-1].reshape(-1, n // (2 * stride), 2, stride)
        values.append(torch.einsum("srp,bgps->bgrs", f, pairs).reshape(-1, n))
    out = torch.stack(values)
    return torch.view_as_real(out) if cplx else out


def butterfly_mult_dyadic_torch(twiddle, input, log_strides, return_intermediates=False):
    """k factors with arbitrary strides, applied in the order given: twiddle
    (nstack, k, n / 2, 2, 2[, 2]), factor i has stride 2^log_strides[i]; input
    (batch, nstack, n[, 2]) (butterfly_multiply.py:733-772).  A debugging aid in the reference
    and here: one PyTorch contraction per factor; with ``return_intermediates`` the input and
    the value after every factor, stacked."""
    cplx = input.dim() == 4
    batch, nstack, n = input.shape[:3]
    _log2(n)
    if twiddle.shape[:5] != (nstack, len(log_strides), n // 2, 2, 2):
        raise ValueError("twiddle must be (nstack, len(log_strides), n / 2, 2, 2) [+ (2,) if complex]")
    x = _as_complex(input) if cplx else input
    t = _as_complex(twiddle) if cplx else twiddle
    values = [x]
    for i, log_stride in enumerate(log_strides):
        stride = 1 << log_stride
        f = t[:, i].reshape(nstack, n // (2 * stride), stride, 2, 2)
        pairs = values[-1].reshape(batch, nstack, n // (2 * stride), 2, stride)
        values.append(torch.einsum("sglrp,bsgpl->bsgrl", f, pairs).reshape(batch, nstack, n))
    out = torch.stack(values) if return_intermediates else values[-1]
    return torch.view_as_real(out) if cplx else out


def butterfly_mult_untied_torch(twiddle, input, increasing_stride=True, return_intermediates=False):
    """``butterfly_mult_untied`` under the name of the reference's plain-PyTorch version
    (butterfly_multiply.py:126-165); ``return_intermediates`` walks the factors one by one."""
    if not return_intermediates:
        return butterfly_mult_untied(twiddle, input, increasing_stride)
    m = _log2(input.shape[2])
    order = list(range(m)) if increasing_stride else list(range(m - 1, -1, -1))
    return butterfly_mult_dyadic_torch(twiddle[:, order], input, order, True)


def butterfly_mult_torch(twiddle, input, increasing_stride=True, return_intermediates=False):
    """Tied weights (butterfly_multiply.py:43-81)."""
    m = _log2(input.shape[2])
    return butterfly_mult_untied_torch(twiddle[:, _tied_index(m, twiddle.device)], input, increasing_stride,
                                       return_intermediates)


def butterfly_mult_conv2d_torch(twiddle, input, kernel_size, padding, increasing_stride=True,
                                return_intermediates=False):
    """(butterfly_multiply.py:491-521)"""
    return butterfly_mult_untied_torch(twiddle, _conv2d_patches(twiddle, input, kernel_size, padding),
                                       increasing_stride, return_intermediates)


def bbt_mult_untied_torch(twiddle, input):
    """(butterfly_multiply.py:377-386)"""
    return bbt_mult_untied(twiddle, input, fast=False)


# The remaining plain-PyTorch twins of the reference compute what the functions above compute.
butterfly_ortho_mult_tied_torch = butterfly_ortho_mult_tied
butterfly_ortho_mult_untied_torch = butterfly_ortho_mult_untied
bbt_ortho_mult_untied_torch = bbt_ortho_mult_untied
bbt_mult_conv2d_torch = bbt_mult_conv2d


def _tied_blocks(factors, m):
    """Tied factors (nstack, nchunks, n - 1, 2, 2), chunk k running with decreasing (even k) or
    increasing (odd k) stride -> (nstack, nchunks, log n, n / 2, 2, 2) in order of application."""
    idx = _tied_index(m, factors.device)
    even = factors[:, 0::2][:, :, idx.flip(0)]
    odd = factors[:, 1::2][:, :, idx]
    return torch.stack((even, odd), 2).reshape(factors.shape[0], factors.shape[1], m, 1 << (m - 1), 2, 2)


def bbt_ortho_mult_tied(twiddle, input):
    """Angles (nstack, nblocks * 2, n - 1): slice 0 of a block with decreasing, slice 1 with
    increasing stride (butterfly_multiply.py:389-398)."""
    if twiddle.shape[1] % 2:
        raise ValueError("twiddle must have shape (nstack, nblocks * 2, n - 1)")
    m = _log2(input.shape[2])
    return _multiply(_tied_blocks(_rotation(twiddle), m), input, False)


def _with_middle_diagonals(blocks, diag):
    """blocks (nstack, nblocks * 2, log n, n / 2, 2, 2) in order of application, diag (nstack,
    nblocks, n): scales the output of every even slice, i.e. the rows of its last factor,
    whose stride is 1 (pair i = elements 2 i, 2 i + 1)."""
    nstack, nchunks, m, half = blocks.shape[:4]
    even = blocks[:, 0::2]
    last = even[:, :, m - 1:] * diag.reshape(nstack, nchunks // 2, 1, half, 2, 1)
    even = torch.cat((even[:, :, :m - 1], last), 2)
    return torch.stack((even, blocks[:, 1::2]), 2).reshape(blocks.shape)


def odo_mult_untied(twiddle, diag, input):
    """Angles (nstack, nblocks * 2 log n, n / 2), diag (nstack, nblocks, n): per block an
    orthogonal butterfly with decreasing stride, the diagonal, an orthogonal butterfly with
    increasing stride, all in storage order (butterfly_multiply.py:452-489; the relation to the
    plain functions is stated in tests_old/test_butterfly_multiply.py:575-579)."""
    m = _log2(input.shape[2])
    nstack = twiddle.shape[0]
    nchunks = twiddle.shape[1] // m
    if nchunks * m != twiddle.shape[1] or nchunks % 2 or nchunks == 0:
        raise ValueError("twiddle must hold nblocks * 2 * log n angle slices, nblocks >= 1")
    blocks = _rotation(twiddle).reshape(nstack, nchunks, m, 1 << (m - 1), 2, 2)
    return _multiply(_with_middle_diagonals(blocks, diag), input, False)


def odo_mult_tied(twiddle, diag, input):
    """The same structure with tied angles (nstack, nblocks * 2, n - 1).  (The reference
    constructs this parameter shape for param='odo' with tied weights but has no kernel that
    accepts it.)"""
    m = _log2(input.shape[2])
    return _multiply(_with_middle_diagonals(_tied_blocks(_rotation(twiddle), m), diag), input, False)


# ---- modules of butterfly/butterfly.py ------------------------------------------------------------

def _stochastic(p):
    return torch.stack((torch.stack((p, 1 - p), -1), torch.stack((1 - p, p), -1)), -2)


class Butterfly(nn.Module):
    """The legacy layer: a product of log n butterfly factors (or of B B^T blocks), usable
    where nn.Linear is (reference: butterfly/butterfly.py:13-330; same constructor arguments,
    parameter names and shapes).

    ``fast`` selects the fast twiddle format where the reference defines it: real, untied,
    param='regular' (any nblocks) and param='odo' (fused ODO blocks).  For the combinations
    whose construction fails in the reference (tied or complex twiddles with fast=True, its
    default) the flag is ignored and the plain format is used."""

    def __init__(self, in_size, out_size, bias=True, complex=False, tied_weight=True, increasing_stride=True,
                 ortho_init=False, param='regular', max_gain=10.0, nblocks=0, diag_constraint=None, expansion=1,
                 diag_init='normal', diag_bookends=False, fast=True):
        super().__init__()
        if param not in ('regular', 'ortho', 'odo', 'obdobt', 'ds', 'logit', 'ortho2'):
            raise ValueError(f"unknown param {param!r}")
        if diag_constraint not in (None, 'positive', 'bounded', 'square'):
            raise ValueError(f"unknown diag_constraint {diag_constraint!r}")
        self.in_size = in_size
        self.m = m = int(math.ceil(math.log2(in_size)))
        self.in_size_extended = size = 1 << m
        self.out_size = out_size
        self.complex = complex
        self.tied_weight = tied_weight
        self.increasing_stride = increasing_stride
        self.ortho_init = ortho_init
        self.param = param
        self.max_gain = max_gain
        self.max_gain_per_factor = max_gain ** (1 / m)
        self.nblocks = nblocks
        self.diag_constraint = diag_constraint
        self.expansion = expansion
        self.diag_init = diag_init
        self.diag_bookends = diag_bookends
        self.nstack = nstack = int(math.ceil(out_size / size)) * expansion
        if nblocks > 0:
            if complex:
                raise ValueError("B B^T blocks are real only; chain two complex layers instead")
            if param != 'odo' and (tied_weight or param not in ('regular', 'ortho', 'obdobt')):
                raise ValueError("B B^T blocks need untied weights and param regular / ortho / odo / obdobt")
        if param != 'regular' and complex:
            raise ValueError("only param='regular' supports complex")
        if tied_weight:
            core = (nstack, size - 1) if nblocks == 0 else (nstack, nblocks * 2, size - 1)
        else:
            core = (nstack, m, size // 2) if nblocks == 0 else (nstack, nblocks * 2 * m, size // 2)
        self.fast = bool(fast) and ((param == 'regular' and not tied_weight and not complex) or param == 'odo')
        if param == 'regular':
            twiddle = self._regular_init(core)
            if self.fast:
                chunks = []
                for k, chunk in enumerate(twiddle.split(m, dim=1)):
                    f = twiddle_normal_to_fast_format(chunk)
                    # stages in order of application: decreasing stride reverses the slice order
                    decreasing = (not increasing_stride) if nblocks == 0 else k % 2 == 0
                    chunks.append(f.flip(1) if decreasing else f)
                twiddle = torch.cat(chunks, dim=1)
            self.twiddle = nn.Parameter(twiddle)
        else:
            gen = {'normal': torch.randn, 'one': torch.ones,
                   'bernoulli': lambda *shape: (torch.rand(*shape) >= 0.5).float() * 2 - 1}
            if diag_init not in gen:
                raise ValueError(f"diag_init {diag_init!r} not supported")
            make_diag = gen[diag_init]
            angle = lambda: nn.Parameter(torch.rand(core) * math.pi * 2)
            if param == 'odo' and self.fast:
                if nblocks == 0:
                    raise ValueError("param='odo' with fast=True needs nblocks >= 1")
                self.twiddle = angle()
                self.diag = nn.Parameter(make_diag(nstack, nblocks, size))
            elif param == 'ortho':
                self.twiddle = angle()
            elif param == 'odo':
                self.twiddle, self.twiddle1 = angle(), angle()
                self.diag = nn.Parameter(make_diag(nstack, size) / math.sqrt(nstack))
                if diag_bookends:
                    self.diag_l = nn.Parameter(make_diag(nstack, size))
                    self.diag_r = nn.Parameter(make_diag(nstack, size))
            elif param == 'obdobt':
                if tied_weight:
                    raise ValueError("param='obdobt' needs untied weights")
                self.twiddle, self.twiddle1 = angle(), angle()
                self.diag = nn.Parameter(make_diag(core[0], nstack, size))
            elif param == 'ds':
                self.twiddle = nn.Parameter(torch.rand(core))
            elif param == 'logit':
                self.twiddle = nn.Parameter(torch.rand(core) * 2 - 1)
            else:  # ortho2
                self.twiddle = nn.Parameter(torch.rand(core) * 2 * math.pi)
        for name in ('twiddle', 'twiddle1', 'diag', 'diag_l', 'diag_r'):
            if getattr(self, name, None) is not None:
                getattr(self, name)._is_structured = True   # the reference's flag against weight decay
        if bias:
            self.bias = nn.Parameter(torch.empty((out_size,) if not complex else (out_size, 2)))
        else:
            self.register_parameter('bias', None)
        self.reset_parameters()

    def _regular_init(self, core):
        if not self.ortho_init:
            shape = core + ((2, 2, 2) if self.complex else (2, 2))
            return torch.randn(shape) * (0.5 if self.complex else 1.0 / math.sqrt(2))
        if not self.complex:
            # a rotation or a reflection per pair
            theta = torch.rand(core) * math.pi * 2
            c, s = torch.cos(theta), torch.sin(theta)
            det = torch.randint(0, 2, core, dtype=c.dtype) * 2 - 1
            return torch.stack((torch.stack((det * c, -det * s), -1), torch.stack((s, c), -1)), -2)
        # Haar measure on U(2): [[c e^{i(a+psi)}, s e^{i(a+chi)}], [-s e^{i(a-chi)}, c e^{i(a-psi)}]]
        phi = torch.asin(torch.sqrt(torch.rand(core)))
        c, s = torch.cos(phi), torch.sin(phi)
        alpha, psi, chi = torch.rand((3,) + core) * math.pi * 2
        polar = lambda r, t: torch.stack((r * torch.cos(t), r * torch.sin(t)), -1)
        top = torch.stack((polar(c, alpha + psi), polar(s, alpha + chi)), -2)
        bottom = torch.stack((polar(-s, alpha - chi), polar(c, alpha - psi)), -2)
        return torch.stack((top, bottom), -3)

    def reset_parameters(self):
        """Bias as in nn.Linear."""
        if self.bias is not None:
            bound = 1 / math.sqrt(self.in_size)
            nn.init.uniform_(self.bias, -bound, bound)

    def _ortho(self, twiddle, x, increasing_stride):
        """One orthogonal butterfly (or B B^T chain) of the non-fused parameterisations."""
        if self.tied_weight:
            return butterfly_ortho_mult_tied(twiddle, x, increasing_stride) if self.nblocks == 0 \
                else bbt_ortho_mult_tied(twiddle, x)
        return butterfly_ortho_mult_untied(twiddle, x, increasing_stride) if self.nblocks == 0 \
            else bbt_ortho_mult_untied(twiddle, x)

    def forward(self, input):
        """input (batch, *, in_size[, 2]) -> (batch, *, out_size[, 2])."""
        x = self.pre_process(input)
        inc = self.increasing_stride
        if self.param == 'regular':
            if self.tied_weight:
                x = butterfly_mult(self.twiddle, x, inc)
            elif self.nblocks == 0:
                x = butterfly_mult_untied(self.twiddle, x, inc, self.training, self.fast)
            else:
                x = bbt_mult_untied(self.twiddle, x, self.fast)
        elif self.param == 'ortho':
            x = self._ortho(self.twiddle, x, inc)
        elif self.param == 'odo':
            diag = self.diag
            if self.diag_constraint == 'positive':
                with torch.no_grad():
                    diag.clamp_(min=0)
            elif self.diag_constraint == 'bounded':
                with torch.no_grad():
                    diag.clamp_(min=1 / self.max_gain, max=self.max_gain)
            elif self.diag_constraint == 'square':
                diag = diag * diag
            if self.fast:
                x = odo_mult_tied(self.twiddle, diag, x) if self.tied_weight else odo_mult_untied(self.twiddle, diag, x)
            else:
                if self.diag_bookends:
                    x = x * self.diag_r
                x = self._ortho(self.twiddle, x, False if self.tied_weight else inc)
                x = x * diag
                x = self._ortho(self.twiddle1, x, True if self.tied_weight else not inc)
                if self.diag_bookends:
                    x = x * self.diag_l
        elif self.param == 'obdobt':
            for t, t1, d in zip(self.twiddle.split(self.m, dim=1), self.twiddle1.split(self.m, dim=1), self.diag):
                x = butterfly_ortho_mult_untied(t, x, False)
                x = x * d
                x = butterfly_ortho_mult_untied(t1, x, True)
        else:
            if self.param == 'ds':
                p = self.twiddle
            elif self.param == 'logit':
                p = torch.sigmoid(self.twiddle)
            else:
                p = torch.cos(self.twiddle) ** 2
            twiddle = _stochastic(p)
            x = butterfly_mult(twiddle, x, inc) if self.tied_weight else butterfly_mult_untied(twiddle, x, inc)
        return self.post_process(input, x)

    def pre_process(self, input):
        tail = (2,) if self.complex else ()
        x = input.reshape(-1, self.in_size, *tail)
        if self.in_size != self.in_size_extended:
            pad = self.in_size_extended - self.in_size
            x = F.pad(x, (0, 0, 0, pad) if self.complex else (0, pad))
        return x.unsqueeze(1).expand(x.shape[0], self.nstack, self.in_size_extended, *tail)

    def _fold_stacks(self, flat, dim):
        """The stacked outputs side by side along ``dim``: when they cover the (power-of-2
        padded) output at least twice they are summed over, then the first out_size columns
        are kept (butterfly.py:262-276)."""
        total = flat.shape[dim]
        out_ext = 1 << int(math.ceil(math.log2(self.out_size)))
        if total // out_ext >= 2:
            flat = flat.unflatten(dim, (total // out_ext, out_ext)).sum(dim=dim)
        if self.out_size != flat.shape[dim]:
            flat = flat.narrow(dim, 0, self.out_size)
        return flat

    def post_process(self, input, output):
        tail = (2,) if self.complex else ()
        batch = output.shape[0]
        flat = self._fold_stacks(output.reshape(batch, self.nstack * self.in_size_extended, *tail), 1)
        if self.bias is not None:
            flat = flat + self.bias
        lead = input.shape[:-2] if self.complex else input.shape[:-1]
        return flat.reshape(*lead, self.out_size, *tail)

    def extra_repr(self):
        s = (f"in_size={self.in_size}, out_size={self.out_size}, bias={self.bias is not None}, "
             f"complex={self.complex}, tied_weight={self.tied_weight}, increasing_stride={self.increasing_stride}, "
             f"ortho_init={self.ortho_init}, param={self.param}, nblocks={self.nblocks}, "
             f"expansion={self.expansion}, diag_init={self.diag_init}")
        if self.param == 'odo':
            s += f", diag_constraint={'none' if self.diag_constraint is None else self.diag_constraint}"
        return s

    def round_to_perm(self):
        """Snap the doubly-stochastic parameterisations to the nearest permutation factors
        (butterfly.py:284-294)."""
        with torch.no_grad():
            if self.param == 'ds':
                self.twiddle_round = self.twiddle.data
                self.twiddle.data = (self.twiddle_round > 0.5).to(self.twiddle.dtype)
            elif self.param == 'logit':
                self.twiddle_round = torch.sigmoid(self.twiddle.data)
                self.twiddle.data = torch.where(self.twiddle_round > 0.5, 10.0, -10.0).to(self.twiddle.dtype)
            elif self.param == 'ortho2':
                self.twiddle_round = torch.cos(self.twiddle.data) ** 2
                self.twiddle.data = torch.where(self.twiddle_round > 0.5, 0.0, math.pi / 2).to(self.twiddle.dtype)


class ButterflyBmm(Butterfly):
    """``matrix_batch`` independent legacy layers applied to the slices of the second to last
    dimension: input (batch, matrix_batch, in_size[, 2]) -> (batch, matrix_batch, out_size[, 2])
    (reference: butterfly/butterfly.py:298-390)."""

    def __init__(self, in_size, out_size, matrix_batch=1, bias=True, complex=False, tied_weight=True,
                 increasing_stride=True, ortho_init=False, param='regular', max_gain=10.0, nblocks=0,
                 diag_constraint=None, expansion=1, diag_init='one', **extra_args):
        m = int(math.ceil(math.log2(in_size)))
        size = 1 << m
        nstack = int(math.ceil(out_size / size))
        super().__init__(size, size * nstack * matrix_batch, bias, complex, tied_weight, increasing_stride,
                         ortho_init, param, max_gain, nblocks, diag_constraint, expansion, diag_init, **extra_args)
        self.in_size = in_size
        self.out_size = out_size
        self.nstack = nstack * expansion
        self.matrix_batch = matrix_batch
        if self.bias is not None:
            tail = (2,) if complex else ()
            with torch.no_grad():
                kept = self.bias.reshape(matrix_batch, size * nstack, *tail)[:, :out_size].contiguous()
            self.bias = nn.Parameter(kept)

    def pre_process(self, input):
        tail = (2,) if self.complex else ()
        batch = input.shape[0]
        x = input
        if self.in_size != self.in_size_extended:
            pad = self.in_size_extended - self.in_size
            x = F.pad(x, (0, 0, 0, pad) if self.complex else (0, pad))
        x = x.unsqueeze(2).expand(batch, self.matrix_batch, self.nstack, self.in_size_extended, *tail)
        return x.reshape(batch, self.matrix_batch * self.nstack, self.in_size_extended, *tail)

    def post_process(self, input, output):
        tail = (2,) if self.complex else ()
        batch = output.shape[0]
        flat = output.reshape(batch, self.matrix_batch, self.nstack * self.in_size_extended, *tail)
        flat = self._fold_stacks(flat, 2)
        return flat if self.bias is None else flat + self.bias

    def extra_repr(self):
        return f"matrix_batch={self.matrix_batch}, " + super().extra_repr()
