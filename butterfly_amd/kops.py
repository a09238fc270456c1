"""``KOP2d``: a 2-D convolution layer written as K2( K1(x) . Kd(weight) ), three learnable
Kronecker-of-butterflies transforms that start out as the 2-D FFT, its copy for the kernel and
the inverse 2-D FFT, so that the layer starts as a circular convolution
(reference: convolution/models/kops.py)."""
import math

import torch
from torch import nn

from .butterfly import Butterfly
from .combine import TensorProduct
from .complex_utils import Complex2Real, Real2Complex, complex_matmul
from .permutation import bitreversal_permutation


class KOP2d(nn.Module):
    """(batch, in_ch, h, w) -> (batch, out_ch, h, w).

    in_size: (h, w) or one int, powers of 2 for the 'fft' initialisation to be a convolution.
    kernel_size: odd, the spatial support of ``weight`` (out_ch, in_ch, k_h, k_w).
    init: 'fft' (the layer equals nn.Conv2d with circular padding and the flipped weight) or
        'ortho' (random orthogonal / unitary factors).
    nblocks, base: blocks per butterfly and radix (4 converts every butterfly with to_base4).
    zero_pad: with complex factors, centre the kernel by a phase ramp on its transform instead
        of rolling it (shift theorem)."""

    def __init__(self, in_size, in_ch, out_ch, kernel_size, complex=True, init="ortho", nblocks=1, base=2,
                 zero_pad=True):
        super().__init__()
        if init not in ("ortho", "fft"):
            raise ValueError("init must be 'ortho' or 'fft'")
        if init == "fft" and not complex:
            raise ValueError("the fft initialisation needs complex=True")
        if base not in (2, 4):
            raise ValueError("base must be 2 or 4")
        self.in_size = (in_size, in_size) if isinstance(in_size, int) else tuple(in_size)
        self.kernel_size = (kernel_size, kernel_size) if isinstance(kernel_size, int) else tuple(kernel_size)
        self.in_ch, self.out_ch = in_ch, out_ch
        self.complex, self.init, self.nblocks, self.base, self.zero_pad = complex, init, nblocks, base, zero_pad
        self.padding = ((self.kernel_size[0] - 1) // 2, (self.kernel_size[1] - 1) // 2)
        # nn.Conv2d's own initialisation, stored flipped: the layer computes a true convolution
        conv = nn.Conv2d(in_ch, out_ch, self.kernel_size, padding=self.padding, bias=False)
        self.weight = nn.Parameter(conv.weight.detach().flip([-1, -2]).clone())

        h, w = self.in_size

        def transform(increasing_stride, kind):
            return TensorProduct(
                Butterfly(w, w, bias=False, complex=complex, increasing_stride=increasing_stride, init=kind,
                          nblocks=nblocks),
                Butterfly(h, h, bias=False, complex=complex, increasing_stride=increasing_stride, init=kind,
                          nblocks=nblocks))

        forward_kind = "ortho" if init == "ortho" else "fft_no_br"
        inverse_kind = "ortho" if init == "ortho" else "ifft_no_br"
        # decimation in frequency on the way in (outputs in bit-reversed order), decimation in
        # time on the way out (inputs in bit-reversed order): no permutation anywhere
        Kd, K1, K2 = transform(False, forward_kind), transform(False, forward_kind), transform(True, inverse_kind)
        with torch.no_grad():
            # unitary transforms on both sides: the kernel's carries the missing sqrt(h w)
            Kd.map1 *= math.sqrt(w)
            Kd.map2 *= math.sqrt(h)
            if zero_pad and complex:
                # the kernel enters at indices 0..k-1 instead of centred on 0: a shift by the
                # padding, i.e. the phase ramp e^{2 pi i p f / n} on frequency f.  The first block
                # ends with the stride-1 stage, whose output rows 2i, 2i+1 hold the frequencies
                # br(2i), br(2i+1).
                for b, p in ((Kd.map1, self.padding[1]), (Kd.map2, self.padding[0])):
                    n = b.n
                    ramp = torch.exp(2j * math.pi * p / n * torch.arange(n))
                    ramp = ramp[bitreversal_permutation(n, pytorch_format=True)].to(b.twiddle.dtype)
                    b.twiddle[:, 0, -1, :, 0, :] *= ramp[0::2].unsqueeze(-1)
                    b.twiddle[:, 0, -1, :, 1, :] *= ramp[1::2].unsqueeze(-1)
        if base == 4:
            for t in (Kd, K1, K2):
                t.map1, t.map2 = t.map1.to_base4(), t.map2.to_base4()
        if complex:
            Kd, K1, K2 = nn.Sequential(Real2Complex(), Kd), nn.Sequential(Real2Complex(), K1), \
                nn.Sequential(K2, Complex2Real())
        self.Kd, self.K1, self.K2 = Kd, K1, K2

    def forward(self, x):
        x_f = self.K1(x)                 # (batch, in_ch, h, w)
        w_f = self.Kd(self.weight)       # (out_ch, in_ch, h, w)
        # per frequency: (batch, in_ch) @ (in_ch, out_ch)
        prod = complex_matmul(x_f.permute(2, 3, 0, 1), w_f.permute(2, 3, 1, 0)).permute(2, 3, 0, 1)
        return self.K2(prod)
