"""The module layer on the device: Butterfly / ButterflyBase4 as nn.Linear drop-ins and the
closed-form transforms against library routines (the reference's tests/test_butterfly.py
and tests/test_special.py are the model)."""
import math
import sys

import numpy as np
import pytest
import scipy.linalg
import torch

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def close(a, b, rtol=1e-3, atol=1e-5):
    return torch.allclose(a, b, rtol=rtol, atol=atol)


def test_butterfly_shapes_and_matrix_flags():
    import butterfly_amd as bfa
    for in_size, out_size in [(7, 15), (15, 7)]:
        for complex_ in (False, True):
            for nblocks in (1, 2, 3):
                for inc in (True, False):
                    say("module", in_size, out_size, complex_, nblocks, inc)
                    b = bfa.Butterfly(in_size, out_size, True, complex_, inc, "ortho", nblocks).cuda()
                    dtype = torch.complex64 if complex_ else torch.float32
                    x = torch.randn(5, 3, in_size, dtype=dtype, device="cuda")
                    y = b(x)
                    assert y.shape == (5, 3, out_size)
                    # dense matrix through the identity (bias removed)
                    eye = torch.eye(in_size, dtype=dtype, device="cuda")
                    M = (b(eye) - b.bias).t()                       # (out, in)
                    assert close(y, x @ M.t() + b.bias, atol=1e-4)
    # transpose / conjugate flags on a square complex layer
    n = 16
    b = bfa.Butterfly(n, n, False, True, True, "randn", 2).cuda()
    eye = torch.eye(n, dtype=torch.complex64, device="cuda")
    M = b(eye).t()
    assert close(b(eye, transpose=True).t(), M.t(), atol=1e-4)
    assert close(b(eye, conjugate=True).t(), M.conj(), atol=1e-4)
    assert close(b(eye, transpose=True, conjugate=True).t(), M.t().conj(), atol=1e-4)


def test_module_bias_matches_separate_addition():
    """Butterfly folds its bias into the multiply; values and all gradients must equal the
    reference formulation (multiply, flatten, slice, + bias; torch_butterfly/butterfly.py:152-169)."""
    import butterfly_amd as bfa
    from butterfly_amd.multiply import butterfly_multiply
    torch.manual_seed(3)
    for in_size, out_size, complex_, nblocks in [(100, 300, False, 2), (64, 40, True, 1), (4096, 4096, False, 2)]:
        say("module bias", in_size, out_size, complex_, nblocks)
        b = bfa.Butterfly(in_size, out_size, True, complex_, True, "randn", nblocks).cuda()
        dtype = torch.complex64 if complex_ else torch.float32
        x = torch.randn(9, in_size, dtype=dtype, device="cuda", requires_grad=True)
        g = torch.randn(9, out_size, dtype=dtype, device="cuda")
        y = b(x)
        grads = torch.autograd.grad(y, (x, b.twiddle, b.bias), g)
        out_cols = b.out_size if b.nstacks == 1 else None
        z = butterfly_multiply(b.twiddle, b.pre_process(x), b.increasing_stride, out_cols)
        z = z.reshape(9, -1)[:, :out_size] + b.bias
        ref = torch.autograd.grad(z, (x, b.twiddle, b.bias), g)
        assert close(y, z, atol=1e-4)
        for a, r in zip(grads, ref):
            assert close(a, r, rtol=1e-3, atol=1e-4 * max(1.0, r.abs().max().item()))


def test_linear_dropin_of_4096_against_the_oracle():
    """Butterfly(4096, 4096, bias=True, init='ortho', nblocks=2), the nn.Linear drop-in of the
    quoted configurations, at a batch where its backward passes keep two row groups in flight:
    output, d_input, d_twiddle against the CPU oracle, d_bias against numpy's column sum."""
    import butterfly_amd as bfa
    from conftest import rel_err
    from oracle import oracle
    torch.manual_seed(11)
    B, n = 4200, 4096
    layer = bfa.Butterfly(n, n, bias=True, init="ortho", nblocks=2).cuda()
    say("linear drop-in", B, n, "increasing_stride", layer.increasing_stride)
    x = torch.randn(B, n, device="cuda", requires_grad=True)
    g = torch.randn(B, n, device="cuda")
    y = layer(x)
    dx, dtw, db = torch.autograd.grad(y, (x, layer.twiddle, layer.bias), g)
    torch.cuda.synchronize()
    tw = layer.twiddle.detach().cpu().numpy()
    bias = layer.bias.detach().cpu().numpy()
    xh, gh = x.detach().cpu().numpy().reshape(B, 1, n), g.cpu().numpy().reshape(B, 1, n)
    inc = bool(layer.increasing_stride)
    y_ref = oracle.butterfly_fw(tw, xh, inc, None).reshape(B, n) + bias
    assert rel_err(y.detach().cpu().numpy(), y_ref) < 1e-5
    dtw_ref, dx_ref = oracle.butterfly_bw(tw, xh, gh, inc)
    assert rel_err(dx.cpu().numpy(), dx_ref.reshape(B, n)) < 1e-4
    assert rel_err(dtw.cpu().numpy(), dtw_ref) < 1e-4
    assert rel_err(db.cpu().numpy(), gh.reshape(B, n).sum(0, dtype=np.float64).astype(np.float32)) < 1e-4


def test_autograd_through_module_reduces_loss():
    import butterfly_amd as bfa
    torch.manual_seed(0)
    b = bfa.Butterfly(64, 64, True, False, True, "randn", 2).cuda()
    x = torch.randn(256, 64, device="cuda")
    target = torch.randn(256, 64, device="cuda")
    opt = torch.optim.SGD(b.parameters(), lr=1e-2)
    losses = []
    for _ in range(20):
        opt.zero_grad()
        loss = ((b(x) - target) ** 2).mean()
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert losses[-1] < losses[0]


def test_fft_ifft_hadamard_circulant():
    from butterfly_amd import special
    torch.manual_seed(1)
    for n in (2, 8, 256, 4096):
        say("fft", n)
        x = torch.randn(3, n, dtype=torch.complex64, device="cuda")
        for br_first in (True, False):
            for normalized in (False, True):
                f = special.fft(n, normalized=normalized, br_first=br_first).cuda()
                want = torch.fft.fft(x, norm="ortho" if normalized else None)
                assert close(f(x), want, rtol=1e-3, atol=1e-3 * math.sqrt(n)), (n, br_first, normalized)
                fi = special.ifft(n, normalized=normalized, br_first=br_first).cuda()
                want = torch.fft.ifft(x, norm="ortho" if normalized else None)
                assert close(fi(x), want, rtol=1e-3, atol=1e-4), (n, br_first, normalized)
    for n in (2, 16, 512):
        for inc in (True, False):
            h = special.hadamard(n, increasing_stride=inc).cuda()
            x = torch.randn(4, n, device="cuda")
            H = torch.tensor(scipy.linalg.hadamard(n), dtype=torch.float32, device="cuda")
            assert close(h(x), x @ H.t(), atol=1e-3)
    for n in (13, 16):
        for sep in (True, False):
            for transposed in (False, True):
                say("circulant", n, sep, transposed)
                col = torch.randn(n, device="cuda")
                C = torch.tensor(scipy.linalg.circulant(col.cpu().numpy()), device="cuda")
                if transposed:
                    C = C.t()
                m = special.circulant(col, transposed=transposed, separate_diagonal=sep)
                x = torch.randn(3, n, device="cuda")
                assert close(m(x), x @ C.t(), atol=1e-4), (n, sep, transposed)
    col, row = torch.randn(9, device="cuda"), torch.randn(6, device="cuda")
    T = torch.tensor(scipy.linalg.toeplitz(col.cpu().numpy(), row.cpu().numpy()), device="cuda")
    m = special.toeplitz(col, row)
    x = torch.randn(2, 6, device="cuda")
    assert close(m(x), x @ T.t(), atol=1e-4)


def test_fft_headline_complex_against_torch_fft():
    """complex64, n = 4096, normalised DFT twiddles, bit reversal outside the operator."""
    from butterfly_amd import special
    torch.manual_seed(2)
    n, B = 4096, 512
    f = special.fft(n, normalized=True).cuda()
    x = torch.randn(B, n, dtype=torch.complex64, device="cuda", requires_grad=True)
    y = f(x)
    want = torch.fft.fft(x.detach(), norm="ortho")
    err = (y.detach() - want).abs().max().item() / want.abs().max().item()
    say("fft 4096 fwd err", err)
    assert err < 1e-5
    g = torch.randn_like(want)
    (dx,) = torch.autograd.grad(y, x, g)
    # adjoint of the unitary DFT is the inverse DFT
    want_dx = torch.fft.ifft(g, norm="ortho")
    err = (dx - want_dx).abs().max().item() / want_dx.abs().max().item()
    say("fft 4096 bwd err", err)
    assert err < 1e-4


def test_base4_module_equals_base2_module():
    import butterfly_amd as bfa
    torch.manual_seed(3)
    for in_size, out_size, nblocks, complex_ in [(256, 256, 1, False), (100, 300, 2, False), (32, 32, 3, True),
                                                 (128, 128, 2, True)]:
        for inc in (True, False):
            say("base4 module", in_size, out_size, nblocks, complex_, inc)
            b2 = bfa.Butterfly(in_size, out_size, True, complex_, inc, "randn", nblocks).cuda()
            b4 = b2.to_base4()
            assert isinstance(b4, bfa.ButterflyBase4) and not hasattr(b4, "twiddle")
            dtype = torch.complex64 if complex_ else torch.float32
            x = torch.randn(9, in_size, dtype=dtype, device="cuda", requires_grad=True)
            y2, y4 = b2(x), b4(x)
            assert close(y4, y2, atol=1e-4)
            g = torch.randn_like(y2)
            (dx2,) = torch.autograd.grad(y2, x, g)
            (dx4,) = torch.autograd.grad(y4, x, g)
            assert close(dx4, dx2, atol=1e-4)


def test_butterfly_unitary_shapes_unitarity_and_gradients():
    """Model: the reference's tests/test_butterfly.py:212-237 (shapes, B B^H = I), plus the
    angle gradients against autograd through a dense matrix built from the same factors."""
    import butterfly_amd as bfa
    torch.manual_seed(11)
    for in_size, out_size in [(7, 15), (15, 7)]:
        for inc in (True, False):
            for nblocks in (1, 2, 3):
                say("unitary", in_size, out_size, inc, nblocks)
                b = bfa.ButterflyUnitary(in_size, out_size, True, inc, nblocks=nblocks).cuda()
                x = torch.randn(10, in_size, dtype=torch.complex64, device="cuda")
                assert b(x).shape == (10, out_size)
    size = 32
    eye = torch.eye(size, dtype=torch.complex64, device="cuda")
    for inc in (True, False):
        for nblocks in (1, 2, 3):
            b = bfa.ButterflyUnitary(size, size, False, inc, nblocks=nblocks).cuda()
            M = b(eye).t()
            assert close(M @ M.conj().t(), eye, atol=1e-4)
            # transpose and conjugate flags give the inverse of a unitary matrix
            assert close(b(b(eye), transpose=True, conjugate=True), eye, atol=1e-4)
    # gradient w.r.t. the angles: compare with the dense product of the same 2x2 factors
    from butterfly_amd.multiply import butterfly_multiply_torch
    b = bfa.ButterflyUnitary(16, 16, False, True, nblocks=2).cuda()
    x = torch.randn(6, 16, dtype=torch.complex64, device="cuda")
    g = torch.randn(6, 16, dtype=torch.complex64, device="cuda")
    (ga,) = torch.autograd.grad(b(x), b.twiddle, g)
    y_ref = butterfly_multiply_torch(b.effective_twiddle(), x.unsqueeze(1), True).squeeze(1)
    (gr,) = torch.autograd.grad(y_ref, b.twiddle, g)
    assert close(ga, gr, rtol=1e-3, atol=1e-4)


def test_butterfly_bmm_equals_loop_over_layers():
    """Model: tests/test_butterfly.py:239-266."""
    import butterfly_amd as bfa
    torch.manual_seed(12)
    mb = 3
    for in_size, out_size in [(7, 15), (15, 7)]:
        for complex_ in (False, True):
            for inc in (True, False):
                for nblocks in (1, 2, 3):
                    say("bmm", in_size, out_size, complex_, inc, nblocks)
                    bmm = bfa.ButterflyBmm(in_size, out_size, mb, True, complex_, inc, nblocks=nblocks).cuda()
                    dtype = torch.complex64 if complex_ else torch.float32
                    x = torch.randn(10, mb, in_size, dtype=dtype, device="cuda", requires_grad=True)
                    y = bmm(x)
                    assert y.shape == (10, mb, out_size)
                    outs = []
                    layers = []
                    for i in range(mb):
                        tw = bmm.twiddle[i * bmm.nstacks:(i + 1) * bmm.nstacks].detach()
                        layer = bfa.Butterfly(in_size, out_size, True, complex_, inc, init=tw, nblocks=nblocks).cuda()
                        with torch.no_grad():
                            layer.bias.copy_(bmm.bias[i])
                        layers.append(layer)
                        outs.append(layer(x[:, i]))
                    y_loop = torch.stack(outs, 1)
                    assert close(y, y_loop, atol=1e-5)
                    g = torch.randn_like(y)
                    gx, gtw, gb = torch.autograd.grad(y, (x, bmm.twiddle, bmm.bias), g)
                    hx = torch.autograd.grad(y_loop, x, g)[0]
                    assert close(gx, hx, atol=1e-4)
                    for i, layer in enumerate(layers):
                        ht, hb = torch.autograd.grad(layer(x[:, i]), (layer.twiddle, layer.bias), g[:, i])
                        assert close(gtw[i * bmm.nstacks:(i + 1) * bmm.nstacks], ht, atol=1e-4)
                        assert close(gb[i], hb, atol=1e-4)


@pytest.mark.parametrize("chunk", range(3))
def test_random_layer_configurations_match_the_host_path(chunk):
    """Seeded random layers (sizes that need padding, trimming and several stacks, real and
    complex, 1-3 blocks, both stride orders, bias or none; Butterfly, ButterflyBase4, ButterflyBmm,
    ButterflyUnitary) with random forward flags: output and every gradient on the device against
    the same layer on host tensors, whose multiply is the operators' host loop (bit-exact with the
    reference's CPU path).  The device takes the fused routes (bias added by the kernel, d_bias
    summed by the backward kernel), the host the composed ones."""
    import copy
    import butterfly_amd as bfa
    rng = np.random.default_rng(4400 + chunk)
    torch.manual_seed(4400 + chunk)
    for i in range(25):
        kind = str(rng.choice(["butterfly", "butterfly", "base4", "bmm", "unitary"]))
        in_size = int(rng.choice([1, 2, 3, 7, 16, 33, 100, 512, 1000, 1500]))
        out_size = int(rng.choice([1, 5, 16, 40, 130, 700, 2100]))
        cplx = bool(rng.random() < 0.4) or kind == "unitary"
        inc = bool(rng.random() < 0.5)
        nblocks = int(rng.choice([1, 2, 3]))
        bias = bool(rng.random() < 0.6)
        lead = [(4,), (3, 5), (2, 1, 3)][int(rng.integers(0, 3))]
        flags = {}
        if kind in ("butterfly", "unitary") and rng.random() < 0.4:
            flags = {"conjugate": bool(rng.random() < 0.5)}
            if in_size == out_size or rng.random() < 0.3:
                flags["transpose"] = True
        say(f"layer case {chunk}.{i}:", kind, in_size, out_size, cplx, inc, nblocks, bias, lead, flags)
        if kind == "butterfly":
            init = str(rng.choice(["randn", "ortho"]))
            host = bfa.Butterfly(in_size, out_size, bias, cplx, inc, init, nblocks)
        elif kind == "base4":
            host = bfa.ButterflyBase4(in_size, out_size, bias, cplx, inc, "randn", nblocks)
        elif kind == "bmm":
            host = bfa.ButterflyBmm(in_size, out_size, 3, bias, cplx, inc, nblocks=nblocks)
            lead = lead + (3,)
        else:
            host = bfa.ButterflyUnitary(in_size, out_size, bias, inc, nblocks)
        dev_layer = copy.deepcopy(host).cuda()
        dtype = torch.complex64 if cplx else torch.float32
        width = in_size
        if flags.get("transpose"):
            # the transposed layer maps the n-padded output side back: feed what its matrix accepts
            width = min(out_size, host.n) if host.nstacks == 1 else None
        if width is None:
            continue
        x = torch.randn(*lead, width, dtype=dtype)
        xh, xd = x.clone().requires_grad_(), x.cuda().requires_grad_()
        yh, yd = host(xh, **flags), dev_layer(xd, **flags)
        assert yd.shape == yh.shape
        g = torch.randn_like(yh)
        wrt_h = (xh,) + tuple(host.parameters())
        wrt_d = (xd,) + tuple(dev_layer.parameters())
        gh = torch.autograd.grad(yh, wrt_h, g, allow_unused=True)
        gd = torch.autograd.grad(yd, wrt_d, g.cuda(), allow_unused=True)
        scale = max(1.0, yh.abs().max().item())
        assert (yd.cpu() - yh).abs().max().item() <= 1e-4 * scale
        for a, b in zip(gd, gh):
            # (an empty parameter -- the twiddle of a layer of size 1, the 4x4 factors of a layer of
            # size 2 -- may come back as an empty gradient on one side and as None on the other)
            assert (a is None or a.numel() == 0) == (b is None or b.numel() == 0)
            if a is not None and b is not None:
                assert a.shape == b.shape
                if b.numel():
                    assert (a.cpu() - b).abs().max().item() <= 2e-4 * max(1.0, b.abs().max().item())
