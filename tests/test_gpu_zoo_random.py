"""Seeded random layers from the constructors of `special`, the legacy package's layer and KOP2d:
on the device (where the layers fold permutations, diagonals and biases into the kernels) against
the same module on host tensors (where they are composed around the operators' host loop, itself
bit-exact with the reference's CPU path, and which tests/test_host_zoo.py holds against
torch.fft / scipy / nn.Conv at the reference's test sizes): output, input gradient and every
parameter gradient."""
import copy
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def draw_layer(rng):
    """One random layer of the zoo with a matching host input: (name, module, input)."""
    from butterfly_amd import kops, legacy, special
    kind = str(rng.choice(["fft", "ifft", "fft_unitary", "dct", "dst", "hadamard", "hadamard_diagonal", "circulant",
                           "toeplitz", "fastfood", "acdc", "conv1d_single", "conv1d_multi", "fft2d", "ifft2d",
                           "conv2d", "wavelet", "legacy", "legacy", "legacy", "kop"]))
    p2 = int(rng.choice([2, 4, 8, 16, 64, 256, 1024, 2048]))
    anyn = int(rng.choice([3, 5, 13, 16, 27, 100, 300, 1024, 1500]))
    f = lambda: bool(rng.random() < 0.5)
    rt = lambda *s: torch.from_numpy(rng.standard_normal(s).astype(np.float32))
    if kind in ("fft", "ifft"):
        m = getattr(special, kind)(p2, normalized=f(), br_first=f(), with_br_perm=f()); x = torch.randn(5, p2, dtype=torch.complex64)
    elif kind == "fft_unitary":
        m = (special.fft_unitary if f() else special.ifft_unitary)(p2, br_first=f(), with_br_perm=f()); x = torch.randn(5, p2, dtype=torch.complex64)
    elif kind == "dct":
        m = special.dct(p2, type=int(rng.choice([2, 3, 4])), normalized=f()); x = torch.randn(5, p2)
    elif kind == "dst":
        m = special.dst(p2, type=int(rng.choice([2, 4])), normalized=f()); x = torch.randn(5, p2)
    elif kind == "hadamard":
        m = special.hadamard(p2, normalized=f(), increasing_stride=f()); x = torch.randn(5, p2)
    elif kind == "hadamard_diagonal":
        k = int(rng.integers(1, 4))
        m = special.hadamard_diagonal(rt(k, p2), normalized=True, increasing_stride=f(), separate_diagonal=f()); x = torch.randn(5, p2)
    elif kind == "circulant":
        cplx = f(); col = torch.randn(anyn, dtype=torch.complex64 if cplx else torch.float32)
        m = special.circulant(col, transposed=f(), separate_diagonal=f()); x = torch.randn(5, anyn, dtype=col.dtype)
    elif kind == "toeplitz":
        cplx = f(); dt = torch.complex64 if cplx else torch.float32
        n_in = int(rng.choice([3, 11, 38, 200]))
        m = special.toeplitz(torch.randn(anyn, dtype=dt), torch.randn(n_in, dtype=dt), separate_diagonal=f()); x = torch.randn(5, n_in, dtype=dt)
    elif kind == "fastfood":
        m = special.fastfood(rt(p2), rt(p2), rt(p2), torch.from_numpy(rng.permutation(p2)), normalized=True,
                             increasing_stride=f(), separate_diagonal=f()); x = torch.randn(5, p2)
    elif kind == "acdc":
        m = special.acdc(rt(p2), rt(p2), dct_first=f(), separate_diagonal=f()); x = torch.randn(5, p2)
    elif kind == "conv1d_single":
        k = int(rng.choice([1, 3, 5])); n = max(anyn, 8)
        m = special.conv1d_circular_singlechannel(n, rt(1, 1, k), f()); x = torch.randn(5, 1, n)
    elif kind == "conv1d_multi":
        k = int(rng.choice([1, 3, 5])); n = max(min(anyn, 300), 8)
        m = special.conv1d_circular_multichannel(n, rt(4, 3, k)); x = torch.randn(5, 3, n)
    elif kind in ("fft2d", "ifft2d"):
        n1, n2 = int(rng.choice([4, 16, 64])), int(rng.choice([2, 8, 32]))
        m = getattr(special, kind)(n1, n2, normalized=f(), br_first=f(), with_br_perm=f(), flatten=f()); x = torch.randn(3, n2, n1, dtype=torch.complex64)
    elif kind == "conv2d":
        n1, n2 = int(rng.choice([8, 13, 16])), int(rng.choice([8, 27, 32]))
        p2ok = (n1 & (n1 - 1)) == 0 and (n2 & (n2 - 1)) == 0
        m = special.conv2d_circular_multichannel(n1, n2, rt(4, 3, 3, 5), flatten=p2ok and f()); x = torch.randn(2, 3, n2, n1)
    elif kind == "wavelet":
        m = special.wavelet_haar(p2, with_perm=f()); x = torch.randn(5, p2)
    elif kind == "legacy":
        param = str(rng.choice(["regular", "regular", "ortho", "odo", "obdobt", "ds", "logit", "ortho2"]))
        nblocks = int(rng.choice([0, 1, 2])) if param in ("regular", "ortho", "odo", "obdobt") else 0
        if param in ("odo", "obdobt"):
            nblocks = max(nblocks, 1)
        # B B^T blocks exist for untied real weights only
        tied = f() and nblocks == 0
        cplx = f() and param == "regular" and nblocks == 0
        in_size, out_size = int(rng.choice([4, 7, 16, 100, 512])), int(rng.choice([3, 16, 40, 700]))
        m = legacy.Butterfly(in_size, out_size, bias=f(), complex=cplx, tied_weight=tied, increasing_stride=f(),
                             ortho_init=f(), param=param, nblocks=nblocks, expansion=int(rng.choice([1, 1, 2])),
                             diag_init=str(rng.choice(["one", "normal"])), fast=f())
        x = torch.randn(5, in_size, 2) if cplx else torch.randn(5, in_size)
    else:
        hw = (int(rng.choice([8, 16])), int(rng.choice([8, 32])))
        cplx = f()
        init = "fft" if (cplx and f()) else "ortho"
        m = kops.KOP2d(hw, 3, 4, int(rng.choice([1, 3])), complex=cplx, init=init, nblocks=int(rng.choice([1, 2])),
                       base=int(rng.choice([2, 4])), zero_pad=f())
        x = torch.randn(2, 3, *hw)
    return kind, m, x


@pytest.mark.parametrize("chunk", range(4))
def test_random_zoo_layers_match_the_host_path(chunk):
    rng = np.random.default_rng(5500 + chunk)
    torch.manual_seed(5500 + chunk)
    for i in range(30):
        kind, host, x = draw_layer(rng)
        say(f"zoo case {chunk}.{i}:", kind, tuple(x.shape), getattr(host, "extra_repr", lambda: "")()[:160])
        onboard = copy.deepcopy(host).cuda()
        xh, xd = x.clone().requires_grad_(), x.cuda().requires_grad_()
        yh, yd = host(xh), onboard(xd)
        assert yd.shape == yh.shape and yd.dtype == yh.dtype
        g = torch.randn_like(yh)
        ph = [p for p in host.parameters() if p.requires_grad]
        pd = [p for p in onboard.parameters() if p.requires_grad]
        gh = torch.autograd.grad(yh, [xh] + ph, g, allow_unused=True)
        gd = torch.autograd.grad(yd, [xd] + pd, g.cuda(), allow_unused=True)
        scale = max(1.0, yh.abs().max().item())
        assert (yd.cpu() - yh).abs().max().item() <= 2e-4 * scale
        for a, b in zip(gd, gh):
            assert (a is None or a.numel() == 0) == (b is None or b.numel() == 0)
            if a is not None and b is not None and b.numel():
                assert a.shape == b.shape
                assert (a.cpu() - b).abs().max().item() <= 5e-4 * max(1.0, b.abs().max().item())
