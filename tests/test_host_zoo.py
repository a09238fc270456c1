"""The `special` / `combine` constructors on HOST tensors, every flag of every constructor,
against independent libraries (torch.fft, scipy.fft, scipy.linalg, nn.Conv1d / nn.Conv2d with
circular padding) at the sizes and tolerances the reference's own tests use
(tests/test_special.py, tests/test_combine.py, tests/test_butterfly.py: rtol 1e-3, atol 1e-5).
On host tensors the layers run the operators' host loop, so this also holds the modules'
bookkeeping (permutations, diagonals, padding, stacking) apart from any device code."""
import itertools
import math

import numpy as np
import pytest
import scipy.fft
import scipy.linalg as la
import torch
import torch.nn.functional as F
from torch import nn

RTOL, ATOL = 1e-3, 1e-5


def close(a, b, atol=ATOL):
    return torch.allclose(a, b, RTOL, atol)


@pytest.fixture(autouse=True)
def _seed():
    torch.manual_seed(1234)
    np.random.seed(1234)


def test_fourier_1d_every_flag():
    from butterfly_amd import special
    n = 16
    x = torch.randn(10, n, dtype=torch.complex64)
    for normalized, br_first in itertools.product((False, True), (True, False)):
        norm = "ortho" if normalized else None
        assert close(special.fft(n, normalized=normalized, br_first=br_first)(x), torch.fft.fft(x, norm=norm))
        assert close(special.ifft(n, normalized=normalized, br_first=br_first)(x), torch.fft.ifft(x, norm=norm))
    for br_first in (True, False):
        assert close(special.fft_unitary(n, br_first=br_first)(x), torch.fft.fft(x, norm="ortho"))
        assert close(special.ifft_unitary(n, br_first=br_first)(x), torch.fft.ifft(x, norm="ortho"))
    # without the bit reversal the layer is the transform up to that permutation, on the side br_first names
    from butterfly_amd.permutation import bitreversal_permutation
    br = bitreversal_permutation(n, pytorch_format=True)
    for make, ref in ((special.fft, torch.fft.fft), (special.ifft, torch.fft.ifft)):
        for br_first in (True, False):
            b = make(n, normalized=True, br_first=br_first, with_br_perm=False)
            out = b(x[:, br]) if br_first else b(x)[:, br]
            assert close(out, ref(x, norm="ortho"))


def test_trigonometric_transforms_against_scipy():
    from butterfly_amd import special
    n = 16
    x = torch.randn(10, n)
    for kind, normalized in itertools.product((2, 3, 4), (False, True)):
        want = torch.tensor(scipy.fft.dct(x.numpy(), type=kind, norm="ortho" if normalized else None))
        assert close(special.dct(n, type=kind, normalized=normalized)(x), want, 1e-4)
    for kind, normalized in itertools.product((2, 4), (False, True)):
        want = torch.tensor(scipy.fft.dst(x.numpy(), type=kind, norm="ortho" if normalized else None))
        assert close(special.dst(n, type=kind, normalized=normalized)(x), want, 1e-4)


def test_circulant_and_toeplitz_against_scipy():
    from butterfly_amd import special
    for cplx in (False, True):
        dtype = torch.complex64 if cplx else torch.float32
        n = 13
        vec = torch.randn(n, dtype=dtype)
        x = torch.randn(10, n, dtype=dtype)
        C = torch.tensor(la.circulant(vec.numpy()))
        for transposed, separate in itertools.product((False, True), (True, False)):
            b = special.circulant(vec, transposed=transposed, separate_diagonal=separate)
            M = C.T if transposed else C                 # out = M x: x @ M^T
            assert close(b(x), x @ M.T, 1e-4)
        for n_out, n_in in ((13, 38), (27, 11)):
            col, row = torch.randn(n_out, dtype=dtype), torch.randn(n_in, dtype=dtype)
            T = torch.tensor(la.toeplitz(col.numpy(), row.numpy()))
            x = torch.randn(10, n_in, dtype=dtype)
            for separate in (True, False):
                assert close(special.toeplitz(col, row, separate_diagonal=separate)(x), x @ T.T, 1e-4)
        col = torch.randn(9, dtype=dtype)                 # row omitted: the symmetric / Hermitian-free default
        x = torch.randn(4, 9, dtype=dtype)
        want = x @ torch.tensor(la.toeplitz(col.numpy(), col.numpy())).T if not cplx else None
        if want is not None:
            assert close(special.toeplitz(col)(x), want, 1e-4)


def test_hadamard_family():
    from butterfly_amd import special
    n = 16
    H = torch.tensor(la.hadamard(n), dtype=torch.float32)
    x = torch.randn(10, n)
    for inc in (True, False):
        assert close(special.hadamard(n, normalized=True, increasing_stride=inc)(x), x @ H.T / math.sqrt(n))
        assert close(special.hadamard(n, normalized=False, increasing_stride=inc)(x), x @ H.T, 1e-4)
    Hn = H / math.sqrt(n)
    for k in (1, 2, 3):
        signs = torch.randint(0, 2, (k, n)) * 2 - 1.0
        want = x
        for d in signs:
            want = (want * d) @ Hn.T
        for inc, separate in itertools.product((True, False), (True, False)):
            b = special.hadamard_diagonal(signs, normalized=True, increasing_stride=inc, separate_diagonal=separate)
            assert close(b(x), want)
    n = 32
    Hn = torch.tensor(la.hadamard(n), dtype=torch.float32) / math.sqrt(n)
    d1 = torch.randint(0, 2, (n,)) * 2 - 1.0
    d2, d3 = torch.randn(2, n)
    perm = torch.randperm(n)
    x = torch.randn(10, n)
    want = ((((x * d1) @ Hn.T)[:, perm] * d2) @ Hn.T) * d3
    for inc, separate in itertools.product((True, False), (True, False)):
        b = special.fastfood(d1, d2, d3, perm, normalized=True, increasing_stride=inc, separate_diagonal=separate)
        assert close(b(x), want, 1e-4)


def test_acdc_against_scipy():
    from butterfly_amd import special
    n = 32
    x = torch.randn(10, n)
    d1, d2 = torch.randn(2, n)
    for separate in (True, False):
        mid = torch.tensor(scipy.fft.dct(x.numpy(), norm="ortho")) * d1
        want = torch.tensor(scipy.fft.idct(mid.numpy(), norm="ortho")) * d2
        assert close(special.acdc(d1, d2, dct_first=True, separate_diagonal=separate)(x), want, 1e-4)
        mid = torch.tensor(scipy.fft.idct(x.numpy(), norm="ortho")) * d1
        want = torch.tensor(scipy.fft.dct(mid.numpy(), norm="ortho")) * d2
        assert close(special.acdc(d1, d2, dct_first=False, separate_diagonal=separate)(x), want, 1e-4)


def test_circular_convolutions_1d_against_nn_conv1d():
    from butterfly_amd import special
    for n, k in itertools.product((13, 16), (1, 3, 5, 7)):
        conv = nn.Conv1d(1, 1, k, padding=(k - 1) // 2, padding_mode="circular", bias=False)
        x = torch.randn(10, 1, n)
        with torch.no_grad():
            want = conv(x)
            for separate in (True, False):
                assert close(special.conv1d_circular_singlechannel(n, conv.weight, separate)(x), want, 1e-4)
        conv = nn.Conv1d(3, 4, k, padding=(k - 1) // 2, padding_mode="circular", bias=False)
        x = torch.randn(10, 3, n)
        with torch.no_grad():
            assert close(special.conv1d_circular_multichannel(n, conv.weight)(x), conv(x), 1e-4)


def test_fourier_2d_every_flag():
    from butterfly_amd import special
    n1, n2 = 16, 32
    x = torch.randn(6, n2, n1, dtype=torch.complex64)
    for normalized, br_first, flatten in itertools.product((False, True), (True, False), (False, True)):
        norm = "ortho" if normalized else None
        b = special.fft2d(n1, n2, normalized=normalized, br_first=br_first, flatten=flatten)
        assert close(b(x), torch.fft.fftn(x, dim=(-1, -2), norm=norm), 1e-4)
        b = special.ifft2d(n1, n2, normalized=normalized, br_first=br_first, flatten=flatten)
        assert close(b(x), torch.fft.ifftn(x, dim=(-1, -2), norm=norm), 1e-4)
    for br_first in (True, False):
        assert close(special.fft2d_unitary(n1, n2, br_first=br_first)(x), torch.fft.fftn(x, dim=(-1, -2), norm="ortho"), 1e-4)
        assert close(special.ifft2d_unitary(n1, n2, br_first=br_first)(x), torch.fft.ifftn(x, dim=(-1, -2), norm="ortho"), 1e-4)


@pytest.mark.parametrize("n1,n2", [(13, 27), (16, 32)])
def test_circular_convolution_2d_against_nn_conv2d(n1, n2):
    from butterfly_amd import special
    flat_cases = (False, True) if (n1 & (n1 - 1)) == 0 and (n2 & (n2 - 1)) == 0 else (False,)
    x = torch.randn(3, 3, n2, n1)
    for k1, k2 in ((1, 1), (3, 5), (7, 3), (5, 7)):
        conv = nn.Conv2d(3, 4, (k2, k1), padding=((k2 - 1) // 2, (k1 - 1) // 2), padding_mode="circular", bias=False)
        with torch.no_grad():
            want = conv(x)
            for flatten in flat_cases:
                b = special.conv2d_circular_multichannel(n1, n2, conv.weight, flatten=flatten)
                assert close(b(x), want, 1e-4)


def test_wavelet_haar_against_the_direct_recursion():
    """pywt is not installed here: the multilevel Haar decomposition written out directly
    (averages and differences over sqrt(2), coarsest first, as pywt.wavedec orders them)."""
    from butterfly_amd import special
    n = 32
    x = torch.randn(10, n)
    approx, details = x, []
    while approx.shape[-1] > 1:
        even, odd = approx[:, 0::2], approx[:, 1::2]
        details.append((even - odd) / math.sqrt(2))
        approx = (even + odd) / math.sqrt(2)
    want = torch.cat([approx] + details[::-1], dim=-1)
    assert close(special.wavelet_haar(n)(x), want, 1e-4)


def test_wavelet_haar_on_the_example_of_the_pywavelets_manual():
    """Known answer: the PyWavelets manual gives pywt.wavedec([1..8], 'db1', level=2) =
    [5, 13], [-2, -2], [-0.70710678] * 4 (db1 is the Haar wavelet; approximation first, then
    details from coarse to fine, a detail being (even - odd) / sqrt(2)).  wavelet_haar decomposes
    to full depth (reference tests/test_special.py:365-372 compares with pywt.wavedec at its
    default, maximal level), i.e. one more level on [5, 13]: 18 / sqrt(2), -8 / sqrt(2)."""
    from butterfly_amd import special
    x = torch.arange(1.0, 9.0).reshape(1, 8)
    r = math.sqrt(0.5)
    want = torch.tensor([[18 * r, -8 * r, -2.0, -2.0, -r, -r, -r, -r]])
    assert close(special.wavelet_haar(8)(x), want, 1e-5)


def test_combine_constructors_as_the_reference_tests_them():
    import butterfly_amd
    from butterfly_amd import combine
    from butterfly_amd.permutation import FixedPermutation
    Butterfly = butterfly_amd.Butterfly
    for cplx, inc, diag_first, nblocks in itertools.product((False, True), (True, False), (True, False), (1, 2, 3)):
        dtype = torch.complex64 if cplx else torch.float32
        for in_size, out_size in ((9, 15), (15, 9)):
            b = Butterfly(in_size, out_size, bias=False, complex=cplx, increasing_stride=inc, nblocks=nblocks)
            kept = b.twiddle.detach().clone()
            d = torch.randn(in_size if diag_first else out_size, dtype=dtype)
            x = torch.randn(5, in_size, dtype=dtype)
            with torch.no_grad():
                want = b(x * d) if diag_first else b(x) * d
                got = combine.diagonal_butterfly(b, d, diag_first, inplace=False)
                assert got is not b and torch.equal(b.twiddle, kept)
                assert close(got(x), want, 1e-4)
                same = combine.diagonal_butterfly(b, d, diag_first, inplace=True)
                assert same is b and close(b(x), want, 1e-4)
    for cplx, inc1, inc2, nb1, nb2 in itertools.product((False, True), (True, False), (True, False), (1, 2), (1, 2)):
        dtype = torch.complex64 if cplx else torch.float32
        # (the size between the factors is a power of 2, as in the reference's test: a product
        # cannot drop columns in the middle)
        b1 = Butterfly(13, 16, bias=False, complex=cplx, increasing_stride=inc1, nblocks=nb1)
        b2 = Butterfly(16, 15, bias=False, complex=cplx, increasing_stride=inc2, nblocks=nb2)
        x = torch.randn(5, 13, dtype=dtype)
        with torch.no_grad():
            assert close(combine.butterfly_product(b1, b2)(x), b2(b1(x)), 1e-4)
    for cplx, inc in itertools.product((False, True), (True, False)):
        dtype = torch.complex64 if cplx else torch.float32
        b1 = Butterfly(8, 8, bias=False, complex=cplx, increasing_stride=inc)
        b2 = Butterfly(16, 16, bias=False, complex=cplx, increasing_stride=inc)
        x = torch.randn(5, 16, 8, dtype=dtype)
        with torch.no_grad():
            want = combine.TensorProduct(b1, b2)(x)
            got = combine.butterfly_kronecker(b1, b2)(x.reshape(5, 128)).reshape(5, 16, 8)
        assert close(got, want, 1e-4)
        for n, nblocks in itertools.product((16, 64), (1, 2, 3)):
            b = Butterfly(n, n, bias=False, complex=cplx, increasing_stride=inc, nblocks=nblocks)
            y = torch.randn(5, n, dtype=dtype)
            flipped = combine.flip_increasing_stride(b)
            assert flipped[1].increasing_stride == (not inc)
            with torch.no_grad():
                assert close(flipped(y), b(y), 1e-4)
    p1, p2 = FixedPermutation(torch.randperm(8)), FixedPermutation(torch.randperm(4))
    x = torch.randn(3, 4, 8)
    want = combine.TensorProduct(p1, p2)(x)
    assert torch.equal(combine.permutation_kronecker(p1, p2)(x.reshape(3, 32)).reshape(3, 4, 8), want)


def test_layer_grid_of_the_reference_on_host_tensors():
    """Shapes over the reference's grid of sizes, dtypes, stride orders, initialisations and block
    counts; 'ortho' factors have spectral norm 1; transposed / conjugated forward against the
    layer's dense matrix; subtwiddle; scaling by `*=` (tests/test_butterfly.py:24-45, 137-190)."""
    import butterfly_amd
    Butterfly = butterfly_amd.Butterfly
    for (in_size, out_size), cplx, inc, init, nblocks in itertools.product(
            ((7, 15), (15, 7)), (False, True), (True, False), ("randn", "ortho", "identity"), (1, 2, 3)):
        b = Butterfly(in_size, out_size, True, cplx, inc, init, nblocks=nblocks)
        x = torch.randn(10, in_size, dtype=torch.complex64 if cplx else torch.float32)
        assert b(x).shape == (10, out_size)
        if init == "ortho":
            norms = np.linalg.norm(b.twiddle.detach().numpy().reshape(-1, 2, 2), ord=2, axis=(1, 2))
            assert np.allclose(norms, 1, atol=1e-5)
    for cplx, inc, nblocks in itertools.product((False, True), (True, False), (1, 2, 3)):
        dtype = torch.complex64 if cplx else torch.float32
        b = Butterfly(16, 16, bias=False, complex=cplx, increasing_stride=inc, nblocks=nblocks)
        with torch.no_grad():
            M = b(torch.eye(16, dtype=dtype)).t()                  # y = M x
            x = torch.randn(4, 16, dtype=dtype)
            assert close(b(x), x @ M.t(), 1e-4)
            assert close(b(x, transpose=True), x @ M, 1e-4)
            assert close(b(x, conjugate=True), x @ M.conj().t(), 1e-4)
            assert close(b(x, transpose=True, conjugate=True), x @ M.conj(), 1e-4)
            before = b(x)
            b *= 3.0
            assert close(b(x), 3.0 * before, 1e-4)
    for inc in (True, False):
        big = Butterfly(64, 64, bias=False, increasing_stride=inc)
        small = Butterfly(16, 16, bias=False, increasing_stride=inc)
        with torch.no_grad():
            small.twiddle.copy_(big.twiddle[:, :, :4, :8] if inc else big.twiddle[:, :, -4:, :8])
            x = torch.randn(3, 16)
            assert close(big(x, subtwiddle=True), small(x), 1e-5)


def test_base4_unitary_and_bmm_layers_on_host_tensors():
    """to_base4 and ButterflyBase4's `*=`, ButterflyUnitary's shapes and unitarity, ButterflyBmm
    against a loop over layers and as a bank of tensor products built with `init=`
    (tests/test_butterfly.py:193-300, tests/test_butterfly_base4.py:19-40)."""
    import butterfly_amd
    from butterfly_amd import combine
    Butterfly, ButterflyBmm = butterfly_amd.Butterfly, butterfly_amd.ButterflyBmm
    grid = itertools.product(((7, 15), (15, 7)), (False, True), (True, False), (1, 2, 3))
    for (in_size, out_size), cplx, inc, nblocks in grid:
        dtype = torch.complex64 if cplx else torch.float32
        x = torch.randn(10, in_size, dtype=dtype)
        with torch.no_grad():
            for init in ("randn", "ortho", "identity"):
                b = Butterfly(in_size, out_size, True, cplx, inc, init, nblocks=nblocks)
                assert close(b.to_base4()(x), b(x), 1e-4)
                b4 = butterfly_amd.ButterflyBase4(in_size, out_size, False, cplx, inc, init, nblocks=nblocks)
                before = b4(x)
                b4 *= 2.75
                assert close(b4(x), 2.75 * before, 1e-4)
            bmm = ButterflyBmm(in_size, out_size, 3, True, cplx, inc, nblocks=nblocks)
            xs = torch.randn(10, 3, in_size, dtype=dtype)
            out = bmm(xs)
            assert out.shape == (10, 3, out_size)
            for i in range(3):
                one = Butterfly(in_size, out_size, True, cplx, inc,
                                init=bmm.twiddle[i * bmm.nstacks:(i + 1) * bmm.nstacks], nblocks=nblocks)
                one.bias.copy_(bmm.bias[i])
                assert close(out[:, i], one(xs[:, i]), 1e-5)
    for (in_size, out_size), inc, nblocks in itertools.product(((7, 15), (15, 7)), (True, False), (1, 2, 3)):
        u = butterfly_amd.ButterflyUnitary(in_size, out_size, True, inc, nblocks=nblocks)
        assert u(torch.randn(10, in_size, dtype=torch.complex64)).shape == (10, out_size)
    for inc, nblocks in itertools.product((True, False), (1, 2, 3)):
        u = butterfly_amd.ButterflyUnitary(32, 32, False, inc, nblocks=nblocks)
        M = u(torch.eye(32, dtype=torch.complex64)).t().detach().numpy()
        assert np.allclose(M @ M.T.conj(), np.eye(32), RTOL, 1e-5)
    # a bank of out_channels x in_channels tensor products as two ButterflyBmm layers
    ci, co, n1, n2 = 2, 3, 16, 8
    x = torch.randn(4, ci, n2, n1, dtype=torch.complex64)
    b1s = [Butterfly(n1, n1, bias=False, complex=True) for _ in range(co * ci)]
    b2s = [Butterfly(n2, n2, bias=False, complex=True) for _ in range(co * ci)]
    with torch.no_grad():
        want = torch.stack([torch.stack([combine.TensorProduct(b1s[o * ci + i], b2s[o * ci + i])(x[:, i])
                                         for i in range(ci)], dim=1) for o in range(co)], dim=1)
        bank1 = ButterflyBmm(n1, n1, matrix_batch=co * ci, bias=False, complex=True,
                             init=torch.cat([b.twiddle for b in b1s]))
        bank2 = ButterflyBmm(n2, n2, matrix_batch=co * ci, bias=False, complex=True,
                             init=torch.cat([b.twiddle for b in b2s]))
        rows = x.transpose(1, 2).reshape(4, n2, 1, ci, n1).expand(4, n2, co, ci, n1).reshape(4, n2, co * ci, n1)
        after1 = bank1(rows)                                     # (batch, n2, co * ci, n1)
        got = bank2(after1.transpose(1, 3)).transpose(1, 3)      # along n2
        got = got.reshape(4, n2, co, ci, n1).permute(0, 2, 3, 1, 4)
    assert close(got, want, 1e-4)
