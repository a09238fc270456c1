"""Closed-form butterflies: FFT / inverse FFT, Hadamard, circulant and Toeplitz multiplies.

Counterparts of the constructors in the reference's torch_butterfly/special.py
(fft :19-49, ifft :90-122, circulant :248-301, toeplitz :304-342, hadamard :345-361).
"""
import math

import torch
from torch import nn
from torch.nn import functional as F

from .butterfly import Butterfly
from .combine import butterfly_product, diagonal_butterfly
from .complex_utils import Complex2Real, Real2Complex, index_last_dim, real2complex
from .diagonal import Diagonal
from .permutation import FixedPermutation, bitreversal_permutation


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
    return nn.Sequential(perm, b) if br_first else nn.Sequential(b, perm)


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
        return nn.Sequential(*core) if was_complex else nn.Sequential(Real2Complex(), *core, Complex2Real())
    with torch.no_grad():
        b_fft = diagonal_butterfly(b_fft, diag, diag_first=False, inplace=True)
    b = butterfly_product(b_fft, b_ifft)
    b.in_size = n
    b.out_size = n
    return b if was_complex else nn.Sequential(Real2Complex(), b, Complex2Real())


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
