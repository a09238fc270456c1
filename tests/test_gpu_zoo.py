"""The closed-form transforms, combinators and permutation tools built on the native multiply,
each against a library routine or a direct computation (the reference's tests/test_special.py,
test_combine.py and test_permutation.py are the model for what is compared)."""
import math
import sys

import numpy as np
import pytest
import scipy.fft
import scipy.linalg
import torch

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def close(a, b, rtol=1e-4, atol=1e-4):
    return torch.allclose(a, b, rtol=rtol, atol=atol)


def crand(*shape):
    return torch.randn(*shape, dtype=torch.complex64, device="cuda")


def test_unitary_fourier_transforms():
    from butterfly_amd import special
    torch.manual_seed(0)
    for n in (2, 16, 64):
        x = crand(5, n)
        for br_first in (True, False):
            say("fft_unitary", n, br_first)
            assert close(special.fft_unitary(n, br_first).cuda()(x), torch.fft.fft(x, norm="ortho"))
            assert close(special.ifft_unitary(n, br_first).cuda()(x), torch.fft.ifft(x, norm="ortho"))


def test_dct_and_dst_against_scipy():
    from butterfly_amd import special
    torch.manual_seed(1)
    for n in (2, 8, 64, 256):
        x = torch.randn(7, n)
        for normalized in (False, True):
            norm = "ortho" if normalized else None
            for t in (2, 3, 4):
                say("dct", n, t, normalized)
                ref = torch.from_numpy(scipy.fft.dct(x.numpy(), type=t, norm=norm))
                out = special.dct(n, type=t, normalized=normalized).cuda()(x.cuda()).cpu()
                assert close(out, ref, rtol=1e-4, atol=1e-4 * max(1.0, ref.abs().max().item()))
            for t in (2, 4):
                say("dst", n, t, normalized)
                ref = torch.from_numpy(scipy.fft.dst(x.numpy(), type=t, norm=norm))
                out = special.dst(n, type=t, normalized=normalized).cuda()(x.cuda()).cpu()
                assert close(out, ref, rtol=1e-4, atol=1e-4 * max(1.0, ref.abs().max().item()))


def test_hadamard_diagonal_and_fastfood():
    from butterfly_amd import special
    torch.manual_seed(2)
    n, k = 32, 3
    H = torch.from_numpy(scipy.linalg.hadamard(n)).float()
    x = torch.randn(6, n)
    diags = torch.randn(k, n)
    for normalized in (False, True):
        Hn = H / math.sqrt(n) if normalized else H
        ref = x
        for d in diags:
            ref = (ref * d) @ Hn.t()
        for inc in (True, False):
            for sep in (True, False):
                say("hadamard_diagonal", normalized, inc, sep)
                m = special.hadamard_diagonal(diags, normalized, inc, sep).cuda()
                assert close(m(x.cuda()).cpu(), ref, atol=1e-3 * ref.abs().max().item())
    d1, d2, d3 = torch.randn(3, n)
    perm = torch.randperm(n)
    for normalized in (False, True):
        Hn = H / math.sqrt(n) if normalized else H
        ref = ((((x * d1) @ Hn.t())[:, perm] * d2) @ Hn.t()) * d3
        for inc in (True, False):
            for sep in (True, False):
                m = special.fastfood(d1, d2, d3, perm, normalized, inc, sep).cuda()
                assert close(m(x.cuda()).cpu(), ref, atol=1e-3 * ref.abs().max().item())


def test_acdc():
    from butterfly_amd import special
    torch.manual_seed(3)
    n = 64
    x = torch.randn(5, n)
    d1, d2 = torch.randn(2, n)
    C = lambda v: torch.from_numpy(scipy.fft.dct(v.numpy(), type=2, norm="ortho"))
    Ci = lambda v: torch.from_numpy(scipy.fft.idct(v.numpy(), type=2, norm="ortho"))
    for dct_first in (True, False):
        ref = Ci(C(x) * d1) * d2 if dct_first else C(Ci(x) * d1) * d2
        for sep in (True, False):
            say("acdc", dct_first, sep)
            m = special.acdc(d1, d2, dct_first, sep).cuda()
            assert close(m(x.cuda()).cpu(), ref, atol=1e-4 * max(1.0, ref.abs().max().item()))


def test_circular_convolutions():
    from butterfly_amd import special
    torch.manual_seed(4)
    for n in (13, 16):
        for k in (1, 3, 5):
            for cplx in (False, True):
                dtype = torch.complex64 if cplx else torch.float32
                say("conv1d", n, k, cplx)
                w = torch.randn(1, 1, k, dtype=dtype)
                x = torch.randn(4, 1, n, dtype=dtype)
                ref = torch.nn.functional.conv1d(torch.nn.functional.pad(x, (k // 2, k // 2), mode="circular"), w)
                for sep in (True, False):
                    m = special.conv1d_circular_singlechannel(n, w, sep).cuda()
                    assert close(m(x.cuda()).cpu(), ref)
                w = torch.randn(3, 2, k, dtype=dtype)
                x = torch.randn(4, 2, n, dtype=dtype)
                ref = torch.nn.functional.conv1d(torch.nn.functional.pad(x, (k // 2, k // 2), mode="circular"), w)
                m = special.conv1d_circular_multichannel(n, w).cuda()
                assert close(m(x.cuda()).cpu(), ref)
    for (n1, n2, flatten) in [(8, 16, False), (8, 16, True), (6, 9, False)]:
        for (k1, k2) in [(3, 3), (5, 1)]:
            say("conv2d", n1, n2, k1, k2, flatten)
            w = torch.randn(3, 2, k2, k1)
            x = torch.randn(4, 2, n2, n1)
            xp = torch.nn.functional.pad(x, (k1 // 2, k1 // 2, k2 // 2, k2 // 2), mode="circular")
            ref = torch.nn.functional.conv2d(xp, w)
            m = special.conv2d_circular_multichannel(n1, n2, w, flatten=flatten).cuda()
            assert close(m(x.cuda()).cpu(), ref, atol=1e-3)


def test_fourier_2d():
    from butterfly_amd import special
    torch.manual_seed(5)
    n1, n2 = 16, 8
    x = crand(3, n2, n1)
    for normalized in (False, True):
        norm = "ortho" if normalized else None
        for br_first in (True, False):
            for flatten in (False, True):
                say("fft2d", normalized, br_first, flatten)
                f = special.fft2d(n1, n2, normalized, br_first, flatten=flatten).cuda()
                assert close(f(x), torch.fft.fftn(x, dim=(-2, -1), norm=norm), atol=1e-3)
                f = special.ifft2d(n1, n2, normalized, br_first, flatten=flatten).cuda()
                assert close(f(x), torch.fft.ifftn(x, dim=(-2, -1), norm=norm), atol=1e-3)
    for br_first in (True, False):
        assert close(special.fft2d_unitary(n1, n2, br_first).cuda()(x), torch.fft.fftn(x, dim=(-2, -1), norm="ortho"))
        assert close(special.ifft2d_unitary(n1, n2, br_first).cuda()(x), torch.fft.ifftn(x, dim=(-2, -1), norm="ortho"))


def haar_direct(x):
    """Multilevel orthonormal Haar transform, coarsest first (what pywt.wavedec(x, 'haar')
    returns, concatenated)."""
    out = []
    a = x
    while a.shape[-1] > 1:
        even, odd = a[..., 0::2], a[..., 1::2]
        out.append((even - odd) / math.sqrt(2))
        a = (even + odd) / math.sqrt(2)
    return np.concatenate([a] + out[::-1], axis=-1)


def test_wavelet_haar():
    from butterfly_amd import special
    rng = np.random.default_rng(6)
    for n in (2, 8, 32):
        x = rng.standard_normal((4, n)).astype(np.float32)
        out = special.wavelet_haar(n).cuda()(torch.from_numpy(x).cuda()).detach().cpu().numpy()
        assert np.allclose(out, haar_direct(x), atol=1e-5)


def test_kronecker_and_flip():
    import butterfly_amd as bfa
    from butterfly_amd import combine
    torch.manual_seed(7)
    for cplx in (False, True):
        dtype = torch.complex64 if cplx else torch.float32
        for inc in (True, False):
            say("kronecker", cplx, inc)
            b1 = bfa.Butterfly(8, 8, bias=False, complex=cplx, increasing_stride=inc).cuda()
            b2 = bfa.Butterfly(16, 16, bias=False, complex=cplx, increasing_stride=inc).cuda()
            x = torch.randn(3, 16, 8, dtype=dtype, device="cuda")
            ref = combine.TensorProduct(b1, b2)(x)
            bk = combine.butterfly_kronecker(b1, b2).cuda()
            assert close(bk(x.reshape(3, -1)).reshape(3, 16, 8), ref)
            for nblocks in (1, 2, 3):
                b = bfa.Butterfly(32, 32, bias=False, complex=cplx, increasing_stride=inc, nblocks=nblocks).cuda()
                y = torch.randn(5, 32, dtype=dtype, device="cuda")
                assert close(combine.flip_increasing_stride(b).cuda()(y), b(y))
    p1 = bfa.permutation.FixedPermutation(torch.randperm(8))
    p2 = bfa.permutation.FixedPermutation(torch.randperm(4))
    z = torch.randn(2, 4, 8)
    assert torch.equal(combine.permutation_kronecker(p1, p2)(z.reshape(2, -1)).reshape(2, 4, 8),
                       combine.TensorProduct(p1, p2)(z))


def test_perm2butterfly():
    from butterfly_amd import permutation
    rng = np.random.default_rng(8)
    for n in (2, 3, 13, 64, 200):
        for inc in (False, True):
            for cplx in (False, True):
                v = rng.permutation(n)
                say("perm2butterfly", n, inc, cplx)
                b = permutation.perm2butterfly(v, complex=cplx, increasing_stride=inc).cuda()
                dtype = torch.complex64 if cplx else torch.float32
                x = torch.randn(4, n, dtype=dtype, device="cuda")
                assert torch.equal(b(x), x[:, torch.from_numpy(v).cuda()])
    m = permutation.perm_vec_to_mat(np.array([2, 0, 1]))
    assert np.array_equal(permutation.perm_mat_to_vec(m), [2, 0, 1])
    f = np.kron(np.eye(2), np.array([[1, 0, 2, 0], [0, 3, 0, 4], [5, 0, 6, 0], [0, 7, 0, 8]]))
    assert permutation.is_butterfly_factor(f, 4) and not permutation.is_butterfly_factor(f, 2)
    tw = permutation.matrix_to_butterfly_factor(f, 2, check_input=True)
    assert tw.shape == (4, 2, 2) and np.array_equal(tw[0], [[1, 2], [5, 6]]) and np.array_equal(tw[1], [[3, 4], [7, 8]])
    assert np.array_equal(permutation.wavelet_permutation(8), [0, 4, 2, 6, 1, 3, 5, 7])


def test_kop2d_fft_init_is_a_circular_convolution():
    """Model: convolution/models/test_kops.py of the reference."""
    from butterfly_amd.kops import KOP2d
    torch.manual_seed(9)
    in_ch, out_ch = 3, 6
    for in_size in [(32, 32), (16, 16), (32, 16), (16, 32)]:
        for nblocks in (1, 2, 3):
            for base in (2, 4):
                say("kop2d", in_size, nblocks, base)
                kop = KOP2d(in_size, in_ch, out_ch, 5, init="fft", nblocks=nblocks, base=base).cuda()
                x = torch.randn(10, in_ch, *in_size, device="cuda")
                conv = torch.nn.Conv2d(in_ch, out_ch, 5, padding=2, padding_mode="circular", bias=False).cuda()
                with torch.no_grad():
                    conv.weight.copy_(kop.weight.flip([-1, -2]))
                assert close(kop(x), conv(x), rtol=1e-4, atol=1e-4)
    # gradients reach the kernel and the factors
    kop = KOP2d(16, 2, 3, 3, init="ortho").cuda()
    y = kop(torch.randn(4, 2, 16, 16, device="cuda"))
    y.square().mean().backward()
    assert kop.weight.grad is not None and all(p.grad is not None for p in kop.parameters())


def test_fused_sequential_equals_separate_permutations():
    """FusedSequential (permutations applied by the Butterfly's kernels) against the same
    children run one after the other, forward and gradients, and against torch.fft."""
    from torch import nn
    from butterfly_amd import Butterfly, special, combine
    from butterfly_amd.permutation import FixedPermutation, FusedSequential
    torch.manual_seed(3)

    def compare(fused, x, with_params=True):
        plain = nn.Sequential(*fused)
        assert isinstance(fused, FusedSequential)
        xa = x.clone().requires_grad_()
        xb = x.clone().requires_grad_()
        ya, yb = fused(xa), plain(xb)
        assert close(ya, yb)
        g = torch.randn_like(ya)
        params = [p for p in fused.parameters()] if with_params else []
        ga = torch.autograd.grad(ya, [xa] + params, g)
        gb = torch.autograd.grad(yb, [xb] + params, g)
        for a, b in zip(ga, gb):
            assert close(a, b, rtol=1e-3, atol=1e-3)
        return ya

    for n in (8, 256, 1024, 2048):
        x = crand(33, n)
        for br_first in (True, False):
            say("fused fft", n, br_first)
            y = compare(special.fft(n, br_first=br_first).cuda(), x)
            assert close(y, torch.fft.fft(x), rtol=1e-3, atol=1e-3 * math.sqrt(n))
    say("fused wavelet")
    compare(special.wavelet_haar(64).cuda(), torch.randn(9, 64, device="cuda"))
    say("fused flip")
    b = Butterfly(128, 128, bias=False, increasing_stride=True).cuda()
    flipped = combine.flip_increasing_stride(b).cuda()
    xr = torch.randn(12, 128, device="cuda")
    assert close(compare(flipped, xr), b(xr))
    say("fused, several stacks, bias, odd sizes")
    layer = Butterfly(100, 300, bias=True).cuda()      # n = 128, 3 stacks: only the front folds
    seq = FusedSequential(FixedPermutation(torch.randperm(100)), layer, FixedPermutation(torch.randperm(300))).cuda()
    compare(seq, torch.randn(7, 100, device="cuda"))
    layer = Butterfly(100, 90, bias=True, nblocks=2).cuda()   # one stack: both fold, trimmed output
    seq = FusedSequential(FixedPermutation(torch.randperm(100)), layer, FixedPermutation(torch.randperm(90))).cuda()
    compare(seq, torch.randn(7, 100, device="cuda"))
    say("transpose swaps the tables")
    p_in, q = torch.randperm(128).cuda(), torch.randperm(128).cuda()
    sq = Butterfly(128, 128, bias=False, complex=True).cuda()
    fp, fq = FixedPermutation(p_in), FixedPermutation(q)
    xc = crand(5, 128)
    # matrix M = Q B P (P, Q the gathers); M^T x = P^T B^T Q^T x
    eye = torch.eye(128, dtype=torch.complex64, device="cuda")
    M = fq(sq(fp(eye))).T                          # columns M e_j
    got = sq(xc, transpose=True, in_perm=fp.column_table(128, False), out_index=fq.column_table(128, True))
    assert close(got, xc @ M, rtol=1e-3, atol=1e-3)


def test_fused_sequential_folds_diagonals():
    """A Diagonal next to a Butterfly inside a FusedSequential is multiplied into the layer's
    first / last factor; outputs and every gradient (input, factors, diagonals, bias) must
    match the same children run one after the other."""
    from torch import nn
    from butterfly_amd import Butterfly, special
    from butterfly_amd.diagonal import Diagonal
    from butterfly_amd.permutation import FixedPermutation, FusedSequential
    torch.manual_seed(5)
    calls = []

    def compare(fused, x, folded_layers):
        plain = nn.Sequential(*fused)
        hooks = [m.register_forward_hook(lambda mod, a, o: calls.append(type(mod).__name__)) for m in fused]
        xa = x.clone().requires_grad_()
        xb = x.clone().requires_grad_()
        calls.clear()
        ya = fused(xa)
        assert calls.count("Diagonal") == 0 and calls.count("Butterfly") == folded_layers, calls
        yb = plain(xb)
        for h in hooks:
            h.remove()
        assert close(ya, yb, rtol=1e-4, atol=1e-4)
        g = torch.randn_like(ya)
        params = list(fused.parameters())
        ga = torch.autograd.grad(ya, [xa] + params, g)
        gb = torch.autograd.grad(yb, [xb] + params, g)
        for a, b in zip(ga, gb):
            assert close(a, b, rtol=1e-3, atol=1e-3)

    for n, nblocks, inc, cplx in [(8, 1, True, False), (64, 2, False, False), (1024, 2, False, False),
                                  (256, 3, True, True), (2048, 1, False, False), (2, 1, True, True)]:
        say("diagonal fold", n, nblocks, inc, cplx)
        layer = Butterfly(n, n, bias=False, complex=cplx, increasing_stride=inc, nblocks=nblocks).cuda()
        seq = FusedSequential(Diagonal(n, complex=cplx), layer, Diagonal(n, complex=cplx)).cuda()
        x = crand(19, n) if cplx else torch.randn(19, n, device="cuda")
        compare(seq, x, 1)
    say("diagonals inside permutations, real diagonal on a complex layer")
    layer = Butterfly(128, 128, bias=False, complex=True, nblocks=2).cuda()
    seq = FusedSequential(FixedPermutation(torch.randperm(128)), Diagonal(128), layer,
                          Diagonal(128, complex=True), FixedPermutation(torch.randperm(128))).cuda()
    compare(seq, crand(6, 128), 1)
    say("odd sizes, stacks, bias in front of the second diagonal")
    layer = Butterfly(100, 300, bias=False).cuda()        # n = 128, 3 stacks: both diagonals fold
    seq = FusedSequential(Diagonal(100), layer, Diagonal(300)).cuda()
    compare(seq, torch.randn(7, 100, device="cuda"), 1)
    layer = Butterfly(100, 90, bias=True).cuda()          # bias: only the front diagonal folds
    seq = FusedSequential(Diagonal(100), layer, Diagonal(90)).cuda()
    plain = nn.Sequential(*seq)
    x = torch.randn(7, 100, device="cuda")
    assert close(seq(x), plain(x), rtol=1e-4, atol=1e-4)
    say("chains of layers")
    h = special.hadamard_diagonal(torch.randn(3, 64).sign(), normalized=True, separate_diagonal=True).cuda()
    assert isinstance(h, FusedSequential)
    compare(h, torch.randn(11, 64, device="cuda"), 3)
    say("the layer's own arguments")
    layer = Butterfly(64, 64, bias=True).cuda()
    with pytest.raises(ValueError):
        layer(torch.randn(2, 64, device="cuda"), out_scale=torch.ones(64, device="cuda"))
    with pytest.raises(ValueError):
        layer(torch.randn(2, 64, device="cuda"), transpose=True, in_scale=torch.ones(64, device="cuda"))
