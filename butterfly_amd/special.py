"""Closed-form butterflies: Fourier, cosine / sine, Hadamard and Haar transforms, circulant,
Toeplitz and circular-convolution multiplies, Fastfood and ACDC layers.

Counterparts of the constructors in the reference's torch_butterfly/special.py; every module
returned runs on the native multiply through ``Butterfly`` / ``ButterflyUnitary``.
"""
import math
from functools import reduce

import torch
from torch import nn
from torch.nn import functional as F

from .butterfly import Butterfly, ButterflyUnitary
from .combine import (TensorProduct, butterfly_kronecker, butterfly_product, diagonal_butterfly,
                      permutation_kronecker)
from .complex_utils import Complex2Real, Real2Complex, index_last_dim, real2complex
from .diagonal import Diagonal
from .permutation import FixedPermutation, FusedSequential, bitreversal_permutation, invert, wavelet_permutation


def _log2_exact(n):
    log_n = int(n).bit_length() - 1
    if n != 1 << log_n:
        raise ValueError("n must be a power of 2")
    return log_n


def _dft_twiddle(n, sign):
    """Cooley-Tukey (decimation-in-time) factors, stage idx combining blocks of 2^(idx+1):
    pair i has w = exp(sign 2 pi i k / 2^(idx+1)), k = i mod 2^idx, factor [[1, w], [1, -w]]."""
    log_n = _log2_exact(n)
    stages = []
    for idx in range(log_n):
        size = 2 << idx
        k = torch.arange(n // 2) % (size // 2)
        w = torch.polar(torch.ones(n // 2), sign * 2 * math.pi * k.to(torch.float32) / size)
        one = torch.ones_like(w)
        stages.append(torch.stack((torch.stack((one, w), -1), torch.stack((one, -w), -1)), -2))
    return torch.stack(stages).reshape(1, 1, log_n, n // 2, 2, 2)


def _fourier(n, sign, scale, br_first, with_br_perm):
    twiddle = _dft_twiddle(n, sign)
    if not br_first:
        # decimation in frequency: transpose of the decimation-in-time factorisation
        twiddle = twiddle.transpose(-1, -2).flip([2])
    twiddle = (twiddle * scale).contiguous()
    b = Butterfly(n, n, bias=False, complex=True, increasing_stride=br_first, init=twiddle)
    if not with_br_perm:
        return b
    perm = FixedPermutation(bitreversal_permutation(n, pytorch_format=True))
    return FusedSequential(perm, b) if br_first else FusedSequential(b, perm)


def fft(n, normalized=False, br_first=True, with_br_perm=True) -> nn.Module:
    """Module computing the length-n DFT.  normalized: unitary scaling 1/sqrt(n).
    br_first: bit reversal then increasing-stride butterfly (decimation in time); otherwise
    decreasing-stride butterfly then bit reversal.  with_br_perm=False returns only the
    butterfly."""
    scale = 1 / math.sqrt(2) if normalized else 1.0
    return _fourier(n, -1.0, scale, br_first, with_br_perm)


def ifft(n, normalized=False, br_first=True, with_br_perm=True) -> nn.Module:
    """Module computing the inverse DFT (1/n scaling, or 1/sqrt(n) when normalized)."""
    scale = 1 / math.sqrt(2) if normalized else 0.5
    return _fourier(n, 1.0, scale, br_first, with_br_perm)


def hadamard(n, normalized=False, increasing_stride=True) -> Butterfly:
    """Butterfly computing the (Sylvester-ordered) Hadamard transform of size n."""
    log_n = _log2_exact(n)
    h = torch.tensor([[1.0, 1.0], [1.0, -1.0]])
    if normalized:
        h = h / math.sqrt(2)
    twiddle = h.expand(1, 1, log_n, n // 2, 2, 2).contiguous()
    return Butterfly(n, n, bias=False, increasing_stride=increasing_stride, init=twiddle)


def circulant(col, transposed=False, separate_diagonal=True) -> nn.Module:
    """Module multiplying by the circulant matrix with first column ``col`` (first row when
    transposed): iFFT . diag(FFT(col)) . FFT with the two bit reversals cancelling.  Sizes that
    are not powers of two are embedded in a circulant of twice the next power of two."""
    if col.dim() != 1:
        raise ValueError("col must be a vector")
    was_complex = col.is_complex()
    n = col.shape[0]
    log_n = int(math.ceil(math.log2(n)))
    n_ext = n if n == 1 << log_n else 2 << log_n
    b_fft = fft(n_ext, normalized=True, br_first=False, with_br_perm=False).to(col.device)
    b_fft.in_size = n
    b_ifft = ifft(n_ext, normalized=True, br_first=True, with_br_perm=False).to(col.device)
    b_ifft.out_size = n
    if n < n_ext:
        # [c, 0 ..., c]: the wrapped-around copy completes every row of the small circulant
        col = torch.cat((F.pad(col, (0, 2 * ((1 << log_n) - n))), col))
    if not col.is_complex():
        col = real2complex(col)
    eig = torch.fft.fft(col, norm=None)
    if transposed:
        eig = torch.cat((eig[:1], eig[1:].flip([0])))
    br = bitreversal_permutation(n_ext, pytorch_format=True).to(col.device)
    diag = index_last_dim(eig, br)
    if separate_diagonal:
        core = [b_fft, Diagonal(diagonal_init=diag), b_ifft]
        return FusedSequential(*core) if was_complex else FusedSequential(Real2Complex(), *core, Complex2Real())
    with torch.no_grad():
        b_fft = diagonal_butterfly(b_fft, diag, diag_first=False, inplace=True)
    b = butterfly_product(b_fft, b_ifft)
    b.in_size = n
    b.out_size = n
    return b if was_complex else FusedSequential(Real2Complex(), b, Complex2Real())


def toeplitz(col, row=None, separate_diagonal=True) -> nn.Module:
    """Module multiplying by the Toeplitz matrix with first column ``col`` and first row
    ``row`` (default conj(col); row[0] is ignored), via embedding in a circulant."""
    if row is None:
        row = col.conj()
    if col.dim() != 1:
        raise ValueError("col must be a vector")
    was_complex = col.is_complex()
    (n,), (m,) = col.shape, row.shape
    n_ext = 1 << int(math.ceil(math.log2(n + m - 1)))
    if n + m - 1 < n_ext:
        col = F.pad(col, (0, n_ext - (n + m - 1)))
    col = torch.cat([col, row[1:].flip([0])])
    b = circulant(col, separate_diagonal=separate_diagonal)
    if separate_diagonal:
        first, last = (b[0], b[2]) if was_complex else (b[1], b[3])
    else:
        first = last = b if was_complex else b[1]
    first.in_size = m
    last.out_size = n
    return b


# ---- unitary parameterisation of the Fourier butterflies --------------------------------------

def _fourier_unitary(n, sign, br_first, with_br_perm):
    """ButterflyUnitary equal to the unitary DFT (sign -1) or its inverse (sign +1).

    The decimation-in-time factor [[1, w], [1, -w]] / sqrt 2 with w = e^{i t} is the U(2)
    element [[e^{i(a+p)} c, e^{i(a+x)} s], [-e^{i(a-x)} s, e^{i(a-p)} c]] for c = s = 1/sqrt 2
    (phi = pi/4), a = t/2 + pi/2, p = -a, x = t/2 - pi/2; its transpose [[1, 1], [w, -w]] / sqrt 2
    (decimation in frequency) has the same phi and a with p = x = -a."""
    log_n = _log2_exact(n)
    stages = []
    for idx in range(log_n):
        size = 2 << idx
        k = (torch.arange(n // 2) % (size // 2)).to(torch.float32)
        t = sign * 2 * math.pi * k / size
        alpha = t / 2 + math.pi / 2
        chi = t / 2 - math.pi / 2 if br_first else -alpha
        stages.append(torch.stack((torch.full_like(t, math.pi / 4), alpha, -alpha, chi), -1))
    angles = torch.stack(stages)
    if not br_first:
        angles = angles.flip([0])
    b = ButterflyUnitary(n, n, bias=False, increasing_stride=br_first)
    with torch.no_grad():
        b.twiddle.copy_(angles.reshape(1, 1, log_n, n // 2, 4))
    if not with_br_perm:
        return b
    perm = FixedPermutation(bitreversal_permutation(n, pytorch_format=True))
    return FusedSequential(perm, b) if br_first else FusedSequential(b, perm)


def fft_unitary(n, br_first=True, with_br_perm=True) -> nn.Module:
    """The unitary (1/sqrt n) DFT as a ButterflyUnitary (reference: special.py:52-87)."""
    return _fourier_unitary(n, -1.0, br_first, with_br_perm)


def ifft_unitary(n, br_first=True, with_br_perm=True) -> nn.Module:
    """The unitary inverse DFT as a ButterflyUnitary (reference: special.py:125-161)."""
    return _fourier_unitary(n, 1.0, br_first, with_br_perm)


# ---- cosine and sine transforms ------------------------------------------------------------------

def _even_then_reversed_odd(n):
    """[0, 2, 4, ..., 5, 3, 1]: with v = x[this], element m of v sits at half-sample position
    (4m + 1) / 2 modulo 2n, up to a reflection for the second half."""
    idx = torch.arange(n)
    return torch.cat((idx[::2], idx[1::2].flip([0])))


def _trig_type24(n, sine, shift, normalized):
    """Types II and IV of the DCT / DST from one length-n complex FFT.

    y_k = 2 sum_j x_j trig(pi (k + shift) (2j + 1) / (2n)), trig = cos (shift 0: type II,
    1/2: type IV) or sin (shift 1: type II, 1/2: type IV).  With v = x[evens, reversed odds],
    (2j + 1) / 2 becomes (4m + 1) / 2 for the first half of v and 2n - (4m + 1) / 2 for the
    second, which only changes the sign of the term by s_m = cos(2 pi shift) (cosine) or
    -cos(2 pi shift) (sine) there.  Pulling the phases out of the sum,
        y_k = Re( q_k * FFT_n( p . v )_k ),   p_m = s_m e^{-2 pi i shift m / n},
        q_k = 2 e^{-i pi (k + shift) / (2n)}  (times i for the sine transforms)."""
    m = torch.arange(n, dtype=torch.float32)
    second_half_sign = round(math.cos(2 * math.pi * shift)) * (-1 if sine else 1)
    s_m = torch.where(m < n // 2, torch.ones(n), torch.full((n,), float(second_half_sign)))
    pre = s_m * torch.exp(-2j * math.pi * shift * m / n)
    post = 2 * torch.exp(-1j * math.pi * (m + shift) / (2 * n))
    if sine:
        post = post * 1j
    if normalized:
        # orthonormal rows: 1 / sqrt(2n), and 1 / sqrt(4n) for the one constant-magnitude row of
        # type II (k = 0 for the cosine, k = n - 1 for the sine transform); the unitary FFT
        # already carries 1 / sqrt n
        post = post / math.sqrt(2)
        if shift != 0.5:
            post[n - 1 if sine else 0] /= math.sqrt(2)
    perm = _even_then_reversed_odd(n)
    br = bitreversal_permutation(n, pytorch_format=True)
    b = fft(n, normalized=normalized, br_first=True, with_br_perm=False)
    if sine or shift != 0:
        b = diagonal_butterfly(b, pre[br], diag_first=True)
    b = diagonal_butterfly(b, post, diag_first=False)
    return FusedSequential(FixedPermutation(perm[br]), Real2Complex(), b, Complex2Real())


def dct(n: int, type: int = 2, normalized: bool = False) -> nn.Module:
    """Module computing scipy.fft.dct(x, type, norm='ortho' if normalized else None) for a power
    of 2 n and type 2, 3 or 4 (reference: special.py:164-207).

    Type III is the transpose of type II: y = Re(IFFT-sum(d . x)) scattered back, with
    d_j = c_j e^{i pi j / (2n)}, c_0 = 1, c_j = 2: y_{2m} = v_m, y_{2m+1} = v_{n-1-m}."""
    _log2_exact(n)
    if type not in (2, 3, 4):
        raise ValueError("only DCT types 2, 3 and 4 are supported")
    if type == 2:
        return _trig_type24(n, False, 0.0, normalized)
    if type == 4:
        return _trig_type24(n, False, 0.5, normalized)
    j = torch.arange(n, dtype=torch.float32)
    pre = torch.exp(1j * math.pi * j / (2 * n)) * (math.sqrt(2) if normalized else 2.0)
    pre[0] = 1.0
    b = ifft(n, normalized=normalized, br_first=False, with_br_perm=False)
    if not normalized:
        with torch.no_grad():
            b.twiddle *= 2   # the plain sum, not the 1/n-scaled inverse transform
    b = diagonal_butterfly(b, pre, diag_first=True)
    # the decreasing-stride butterfly leaves v bit-reversed; y = v[inverse of the even/odd order]
    br = bitreversal_permutation(n, pytorch_format=True)
    gather = br[invert(_even_then_reversed_odd(n))]
    return FusedSequential(Real2Complex(), b, Complex2Real(), FixedPermutation(gather))


def dst(n: int, type: int = 2, normalized: bool = False) -> nn.Module:
    """Module computing scipy.fft.dst(x, type, norm='ortho' if normalized else None) for a power
    of 2 n and type 2 or 4 (reference: special.py:210-245)."""
    _log2_exact(n)
    if type not in (2, 4):
        raise ValueError("only DST types 2 and 4 are supported")
    return _trig_type24(n, True, 1.0 if type == 2 else 0.5, normalized)


# ---- Hadamard with diagonals, Fastfood, ACDC ---------------------------------------------------------

def hadamard_diagonal(diagonals: torch.Tensor, normalized: bool = False, increasing_stride: bool = True,
                      separate_diagonal: bool = True) -> nn.Module:
    """x -> H D_k ... H D_2 H D_1 x for the rows D_1..D_k of ``diagonals`` (k, n); the Hadamard
    butterflies alternate stride direction so that they can be merged into one Butterfly when
    separate_diagonal is False (reference: special.py:364-391)."""
    if diagonals.dim() != 2:
        raise ValueError("diagonals must have shape (k, n)")
    n = diagonals.shape[1]
    parts = []
    for i, d in enumerate(diagonals.unbind(0)):
        h = hadamard(n, normalized, increasing_stride != (i % 2 == 1)).to(diagonals.device)
        if separate_diagonal:
            parts += [Diagonal(diagonal_init=d), h]
        else:
            parts.append(diagonal_butterfly(h, d, diag_first=True))
    return FusedSequential(*parts) if separate_diagonal else reduce(butterfly_product, parts)


def fastfood(diag1: torch.Tensor, diag2: torch.Tensor, diag3: torch.Tensor, permutation: torch.Tensor,
             normalized: bool = False, increasing_stride: bool = True,
             separate_diagonal: bool = True) -> nn.Module:
    """x -> D3 H D2 P H D1 x (Fastfood), P the gather x[permutation]
    (reference: special.py:684-711)."""
    (n,) = diag1.shape
    if not (diag2.shape == diag3.shape == permutation.shape == (n,)):
        raise ValueError("diag1, diag2, diag3 and permutation must all have shape (n,)")
    h1 = hadamard(n, normalized, increasing_stride).to(diag1.device)
    h2 = hadamard(n, normalized, not increasing_stride).to(diag1.device)
    if separate_diagonal:
        return FusedSequential(Diagonal(diagonal_init=diag1), h1, FixedPermutation(permutation),
                             Diagonal(diagonal_init=diag2), h2, Diagonal(diagonal_init=diag3))
    h1 = diagonal_butterfly(h1, diag1, diag_first=True)
    h2 = diagonal_butterfly(diagonal_butterfly(h2, diag2, diag_first=True), diag3, diag_first=False)
    return FusedSequential(h1, FixedPermutation(permutation), h2)


def acdc(diag1: torch.Tensor, diag2: torch.Tensor, dct_first: bool = True,
         separate_diagonal: bool = True) -> nn.Module:
    """x -> D2 C^-1 D1 C x (dct_first) or x -> D2 C D1 C^-1 x, C the orthonormal DCT-II and
    C^-1 = C^T the orthonormal DCT-III (reference: special.py:714-779).  Built from the two
    transforms above; with separate_diagonal False the diagonals are folded into the
    neighbouring butterflies where a butterfly is adjacent (they act on real data between a
    Complex2Real and a Real2Complex, so they commute with both)."""
    (n,) = diag1.shape
    if diag2.shape != (n,):
        raise ValueError("diag1 and diag2 must have the same shape (n,)")
    first = dct(n, type=2 if dct_first else 3, normalized=True).to(diag1.device)
    second = dct(n, type=3 if dct_first else 2, normalized=True).to(diag1.device)
    if separate_diagonal:
        return FusedSequential(*first, Diagonal(diagonal_init=diag1), *second, Diagonal(diagonal_init=diag2))
    if dct_first:
        # type II ends [.., butterfly, Complex2Real]; type III ends [.., Complex2Real, permutation]:
        # D1 scales the rows of the first butterfly; D2, moved in front of the closing gather
        # (D P = P D' with D' = D[inverse gather]), scales the rows of the second
        perm, r2c, b1, c2r = first
        r2c2, b2, c2r2, gather = second
        b1 = diagonal_butterfly(b1, diag1.to(b1.twiddle.dtype), diag_first=False)
        moved = diag2[invert(gather.permutation)]
        b2 = diagonal_butterfly(b2, moved.to(b2.twiddle.dtype), diag_first=False)
        return FusedSequential(perm, r2c, b1, c2r, r2c2, b2, c2r2, gather)
    r2c, b1, c2r, gather = first
    perm, r2c2, b2, c2r2 = second
    moved = diag1[invert(gather.permutation)]
    b1 = diagonal_butterfly(b1, moved.to(b1.twiddle.dtype), diag_first=False)
    b2 = diagonal_butterfly(b2, diag2.to(b2.twiddle.dtype), diag_first=False)
    return FusedSequential(r2c, b1, c2r, gather, perm, r2c2, b2, c2r2)


# ---- circular convolutions ----------------------------------------------------------------------

def _conv_column(weight, sizes):
    """First column (per trailing dimension) of the circulant that nn.ConvNd with circular
    padding (k - 1) / 2 applies: cross-correlation, so the kernel is reversed, zero-padded to the
    signal size and rotated so that its centre tap sits at index 0."""
    col = weight
    for dim, n in zip(range(-1, -len(sizes) - 1, -1), sizes):
        k = col.shape[dim]
        if k >= n or k % 2 == 0:
            raise ValueError("kernel sizes must be odd and smaller than the signal")
        pad = [0, 0] * (-dim - 1) + [0, n - k]
        col = F.pad(col.flip([dim]), pad).roll(-(k - 1) // 2, dims=dim)
    return col


def conv1d_circular_singlechannel(n, weight, separate_diagonal=True) -> nn.Module:
    """nn.Conv1d(1, 1, k, padding=(k-1)/2, padding_mode='circular', bias=False) with this
    weight (1, 1, k), as a circulant multiply (reference: special.py:394-413)."""
    if weight.dim() != 3 or tuple(weight.shape[:2]) != (1, 1):
        raise ValueError("weight must have shape (1, 1, kernel_size)")
    return circulant(_conv_column(weight, (n,))[0, 0], separate_diagonal=separate_diagonal)


class DiagonalMultiplySum(nn.Module):
    """(batch, in_channels, *size) -> (batch, out_channels, *size): multiply by a diagonal per
    (out, in) channel pair and sum over the input channels -- the frequency-domain side of a
    multichannel convolution (reference: special.py:417-434)."""

    def __init__(self, diagonal_init):
        super().__init__()
        self.diagonal = nn.Parameter(diagonal_init.detach().clone())
        self.complex = self.diagonal.is_complex()

    def forward(self, input):
        return (input.unsqueeze(1) * self.diagonal).sum(dim=2)


def _extended(n):
    """Transform size for a signal of length n: n itself when it is a power of 2, else twice the
    next power of 2 (room for the wrapped-around copy of the kernel column)."""
    log_n = int(math.ceil(math.log2(n)))
    return n if n == 1 << log_n else 2 << log_n


def _extend_column(col, n, n_ext, dim):
    """[c, 0, ..., 0, c] along ``dim``: the second copy supplies the wrap-around of the length-n
    circulant inside the larger one."""
    if n == n_ext:
        return col
    gap = n_ext - 2 * n
    pad = [0, 0] * (-dim - 1) + [0, gap]
    return torch.cat((F.pad(col, pad), col), dim=dim)


def conv1d_circular_multichannel(n, weight) -> nn.Module:
    """nn.Conv1d(in, out, k, padding=(k-1)/2, padding_mode='circular', bias=False) with this
    weight (out, in, k): FFT, per-frequency channel mixing, inverse FFT; the two bit
    reversals cancel (reference: special.py:437-484)."""
    if weight.dim() != 3:
        raise ValueError("weight must have shape (out_channels, in_channels, kernel_size)")
    was_complex = weight.is_complex()
    col = _conv_column(weight, (n,))
    n_ext = _extended(n)
    b_fft = fft(n_ext, normalized=True, br_first=False, with_br_perm=False).to(col.device)
    b_fft.in_size = n
    b_ifft = ifft(n_ext, normalized=True, br_first=True, with_br_perm=False).to(col.device)
    b_ifft.out_size = n
    col = _extend_column(col, n, n_ext, -1)
    if not col.is_complex():
        col = real2complex(col)
    eig = torch.fft.fft(col, norm=None)   # eigenvalues of the circulants (unnormalised on purpose)
    eig = index_last_dim(eig, bitreversal_permutation(n_ext, pytorch_format=True).to(col.device))
    core = [b_fft, DiagonalMultiplySum(eig), b_ifft]
    return FusedSequential(*core) if was_complex else FusedSequential(Real2Complex(), *core, Complex2Real())


# ---- two-dimensional Fourier transforms and convolutions ---------------------------------------------

def _fourier2d(make, n1, n2, br_first, with_br_perm, flatten, **kwargs):
    b1 = make(n1, br_first=br_first, with_br_perm=False, **kwargs)
    b2 = make(n2, br_first=br_first, with_br_perm=False, **kwargs)
    if flatten and isinstance(b1, ButterflyUnitary):
        raise ValueError("the unitary parameterisation has no Kronecker form")
    b = butterfly_kronecker(b1, b2) if flatten else TensorProduct(b1, b2)
    parts = [b]
    if with_br_perm:
        p1 = FixedPermutation(bitreversal_permutation(n1, pytorch_format=True))
        p2 = FixedPermutation(bitreversal_permutation(n2, pytorch_format=True))
        perm = permutation_kronecker(p1, p2) if flatten else TensorProduct(p1, p2)
        parts = [perm, b] if br_first else [b, perm]
    if flatten:
        return FusedSequential(nn.Flatten(start_dim=-2), *parts, nn.Unflatten(-1, (n2, n1)))
    return parts[0] if len(parts) == 1 else FusedSequential(*parts)


def fft2d(n1: int, n2: int, normalized: bool = False, br_first: bool = True, with_br_perm: bool = True,
          flatten=False) -> nn.Module:
    """torch.fft.fftn over the last two dimensions (n2, n1), as two butterflies (TensorProduct)
    or, with flatten, as one butterfly of size n1 * n2 (reference: special.py:487-515)."""
    return _fourier2d(fft, n1, n2, br_first, with_br_perm, flatten, normalized=normalized)


def ifft2d(n1: int, n2: int, normalized: bool = False, br_first: bool = True, with_br_perm: bool = True,
           flatten=False) -> nn.Module:
    """torch.fft.ifftn over the last two dimensions (reference: special.py:542-570)."""
    return _fourier2d(ifft, n1, n2, br_first, with_br_perm, flatten, normalized=normalized)


def fft2d_unitary(n1: int, n2: int, br_first: bool = True, with_br_perm: bool = True) -> nn.Module:
    """The unitary 2-D DFT from two ButterflyUnitary factors (reference: special.py:518-539)."""
    return _fourier2d(fft_unitary, n1, n2, br_first, with_br_perm, False)


def ifft2d_unitary(n1: int, n2: int, br_first: bool = True, with_br_perm: bool = True) -> nn.Module:
    """The unitary inverse 2-D DFT (reference: special.py:573-594)."""
    return _fourier2d(ifft_unitary, n1, n2, br_first, with_br_perm, False)


def conv2d_circular_multichannel(n1: int, n2: int, weight: torch.Tensor, flatten: bool = False) -> nn.Module:
    """nn.Conv2d(in, out, (k2, k1), padding=((k2-1)/2, (k1-1)/2), padding_mode='circular',
    bias=False) on (batch, in, n2, n1) with this weight (out, in, k2, k1)
    (reference: special.py:597-681).  flatten needs power-of-2 sizes."""
    if weight.dim() != 4:
        raise ValueError("weight must have shape (out_channels, in_channels, k2, k1)")
    was_complex = weight.is_complex()
    col = _conv_column(weight, (n1, n2))
    e1, e2 = _extended(n1), _extended(n2)
    if flatten and (e1 != n1 or e2 != n2):
        raise ValueError("flatten needs n1 and n2 to be powers of 2")
    b_fft = fft2d(e1, e2, normalized=True, br_first=False, with_br_perm=False, flatten=flatten).to(col.device)
    b_ifft = ifft2d(e1, e2, normalized=True, br_first=True, with_br_perm=False, flatten=flatten).to(col.device)
    if flatten:
        b_fft, b_ifft = b_fft[1], b_ifft[1]   # the bare butterflies, without Flatten / Unflatten
    else:
        b_fft.map1.in_size, b_fft.map2.in_size = n1, n2
        b_ifft.map1.out_size, b_ifft.map2.out_size = n1, n2
    col = _extend_column(_extend_column(col, n1, e1, -1), n2, e2, -2)
    if not col.is_complex():
        col = real2complex(col)
    eig = torch.fft.fftn(col, dim=(-2, -1), norm=None)
    br1 = bitreversal_permutation(e1, pytorch_format=True).to(col.device)
    br2 = bitreversal_permutation(e2, pytorch_format=True).to(col.device)
    eig = eig.index_select(-2, br2).index_select(-1, br1)
    if flatten:
        eig = eig.flatten(start_dim=-2)
        core = [nn.Flatten(start_dim=-2), b_fft, DiagonalMultiplySum(eig), b_ifft, nn.Unflatten(-1, (n2, n1))]
    else:
        core = [b_fft, DiagonalMultiplySum(eig), b_ifft]
    return FusedSequential(*core) if was_complex else FusedSequential(Real2Complex(), *core, Complex2Real())


# ---- Haar wavelet ----------------------------------------------------------------------------------

def wavelet_haar(n, with_perm=True) -> nn.Module:
    """Multilevel orthonormal Haar transform, output ordered like pywt.wavedec(x, 'haar')
    concatenated: coarsest average, then details from coarse to fine.

    In place, level l (stride 2^l) replaces the averages at positions 2^{l+1} q and
    2^{l+1} q + 2^l by their sum and difference over sqrt 2: stage l of an increasing-stride
    butterfly with the Hadamard factor on the pairs whose index is a multiple of 2^l and the
    identity elsewhere (reference: special.py:782-805)."""
    log_n = _log2_exact(n)
    had = torch.tensor([[1.0, 1.0], [1.0, -1.0]]) / math.sqrt(2)
    eye = torch.eye(2)
    i = torch.arange(n // 2)
    stages = [torch.where((i % (1 << idx) == 0).reshape(-1, 1, 1), had, eye) for idx in range(log_n)]
    b = Butterfly(n, n, bias=False, increasing_stride=True, init=torch.stack(stages).reshape(1, 1, log_n, n // 2, 2, 2))
    if not with_perm:
        return b
    return FusedSequential(b, FixedPermutation(wavelet_permutation(n, pytorch_format=True)))
