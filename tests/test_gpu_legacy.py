"""The legacy ``butterfly`` package adapter (butterfly_amd/legacy.py) on the device against the
numpy restatement of the legacy functions (oracle/legacy_oracle.py), forward and every gradient,
and the legacy modules the way the reference's tests_old/test_butterfly.py exercises them."""
import itertools
import math
import sys

import numpy as np
import pytest
import torch

from oracle import legacy_oracle as lo

pytestmark = pytest.mark.gpu

FW_TOL = 1e-5   # max |err| / max |ref|, float32 / complex64
BW_TOL = 1e-4


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def rel_err(a, b):
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


def pairs(a):
    """complex numpy array -> legacy (..., 2) float32 tensor on the device."""
    return torch.from_numpy(np.stack((a.real, a.imag), -1).astype(np.float32)).cuda()


def unpairs(t):
    a = t.detach().cpu().numpy().astype(np.float64)
    return a[..., 0] + 1j * a[..., 1]


def dev(a):
    return torch.from_numpy(a.astype(np.float32)).cuda()


def grads(out, wrt, g):
    return torch.autograd.grad(out, wrt, g)


def rnd(rng, shape, cplx=False):
    a = rng.standard_normal(shape)
    return (a + 1j * rng.standard_normal(shape)) / math.sqrt(2) if cplx else a


@pytest.mark.parametrize("n,B,S", [(2, 3, 1), (16, 9, 2), (512, 300, 1), (2048, 20, 1)])
@pytest.mark.parametrize("cplx", [False, True], ids=["real", "complex"])
def test_tied_and_untied_multiply(n, B, S, cplx):
    from butterfly_amd import legacy
    m = n.bit_length() - 1
    rng = np.random.default_rng(100 + n)
    x, g = rnd(rng, (B, S, n), cplx), rnd(rng, (B, S, n), cplx)
    to_dev, back = (pairs, unpairs) if cplx else (dev, lambda t: t.detach().cpu().numpy().astype(np.float64))
    for inc in (True, False):
        say("legacy tied/untied", n, B, S, cplx, inc)
        tied = rnd(rng, (S, n - 1, 2, 2), cplx) / math.sqrt(2)
        y_ref, dtw_ref, dx_ref = lo.butterfly_mult(tied, x, inc, g)
        tw_d, x_d = to_dev(tied).requires_grad_(), to_dev(x).requires_grad_()
        y = legacy.butterfly_mult(tw_d, x_d, inc)
        dtw, dx = grads(y, (tw_d, x_d), to_dev(g))
        assert rel_err(back(y), y_ref) < FW_TOL
        assert rel_err(back(dx), dx_ref) < BW_TOL
        assert rel_err(back(dtw), dtw_ref) < BW_TOL
        untied = rnd(rng, (S, m, n // 2, 2, 2), cplx) / math.sqrt(2)
        y_ref, dtw_ref, dx_ref = lo.butterfly_mult_untied(untied, x, inc, g)
        tw_d, x_d = to_dev(untied).requires_grad_(), to_dev(x).requires_grad_()
        y = legacy.butterfly_mult_untied(tw_d, x_d, inc)
        dtw, dx = grads(y, (tw_d, x_d), to_dev(g))
        assert rel_err(back(y), y_ref) < FW_TOL
        assert rel_err(back(dx), dx_ref) < BW_TOL
        assert rel_err(back(dtw), dtw_ref) < BW_TOL


@pytest.mark.parametrize("n,B,S", [(8, 5, 2), (512, 2048, 1)])
def test_fast_format(n, B, S):
    """The fast-format entries against the relations the reference's tests state
    (tests_old/test_butterfly_multiply.py:335-366 and 441-470)."""
    from butterfly_amd import legacy
    m = n.bit_length() - 1
    rng = np.random.default_rng(200 + n)
    x, g = rnd(rng, (B, S, n)), rnd(rng, (B, S, n))
    tw = rnd(rng, (S, m, n // 2, 2, 2)) / math.sqrt(2)
    fast = lo.twiddle_normal_to_fast_format(tw)
    assert np.array_equal(legacy.twiddle_normal_to_fast_format(dev(tw)).cpu().numpy(), fast.astype(np.float32))
    for inc in (True, False):
        say("legacy fast", n, inc)
        f = np.ascontiguousarray(fast if inc else fast[:, ::-1])
        y_ref, df_ref, dx_ref = lo.butterfly_mult_untied_fast(f, x, inc, g)
        f_d, x_d = dev(f).requires_grad_(), dev(x).requires_grad_()
        y = legacy.butterfly_mult_untied(f_d, x_d, inc, True, True)
        df, dx = grads(y, (f_d, x_d), dev(g))
        assert rel_err(y.detach().cpu().numpy(), y_ref) < FW_TOL
        assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
        assert rel_err(df.cpu().numpy(), df_ref) < BW_TOL
    nblocks = 3
    say("legacy bbs fast", n)
    f = rnd(rng, (S, nblocks * 2 * m, 2, n)) / math.sqrt(2)
    y_ref, df_ref, dx_ref = lo.bbt_mult_untied_fast(f, x, g)
    f_d, x_d = dev(f).requires_grad_(), dev(x).requires_grad_()
    y = legacy.bbt_mult_untied(f_d, x_d, True)
    df, dx = grads(y, (f_d, x_d), dev(g))
    assert rel_err(y.detach().cpu().numpy(), y_ref) < FW_TOL
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(df.cpu().numpy(), df_ref) < BW_TOL


@pytest.mark.parametrize("n,B,S", [(4, 3, 2), (64, 40, 2), (512, 600, 1)])
def test_orthogonal_bbt_and_odo(n, B, S):
    from butterfly_amd import legacy
    m = n.bit_length() - 1
    rng = np.random.default_rng(300 + n)
    x, g = rnd(rng, (B, S, n)), rnd(rng, (B, S, n))
    x_d = dev(x).requires_grad_()
    out = lambda t: t.detach().cpu().numpy()

    def check(got, ref, names):
        for (a, b, name) in zip(got, ref, names):
            tol = FW_TOL if name == "y" else BW_TOL
            assert rel_err(out(a), b) < tol, (name, rel_err(out(a), b))

    for inc in (True, False):
        say("legacy ortho", n, inc)
        th = rng.uniform(0, 2 * np.pi, (S, n - 1))
        th_d = dev(th).requires_grad_()
        y = legacy.butterfly_ortho_mult_tied(th_d, x_d, inc)
        check((y,) + grads(y, (th_d, x_d), dev(g)), lo.butterfly_ortho_mult_tied(th, x, inc, g), ("y", "d_theta", "d_x"))
        th = rng.uniform(0, 2 * np.pi, (S, m, n // 2))
        th_d = dev(th).requires_grad_()
        y = legacy.butterfly_ortho_mult_untied(th_d, x_d, inc)
        check((y,) + grads(y, (th_d, x_d), dev(g)), lo.butterfly_ortho_mult_untied(th, x, inc, g), ("y", "d_theta", "d_x"))
    nblocks = 2
    say("legacy bbt", n)
    tw = rnd(rng, (S, nblocks * 2 * m, n // 2, 2, 2)) / math.sqrt(2)
    tw_d = dev(tw).requires_grad_()
    y = legacy.bbt_mult_untied(tw_d, x_d, fast=False)
    check((y,) + grads(y, (tw_d, x_d), dev(g)), lo.bbt_mult_untied(tw, x, g), ("y", "d_tw", "d_x"))
    th = rng.uniform(0, 2 * np.pi, (S, nblocks * 2 * m, n // 2))
    th_d = dev(th).requires_grad_()
    y = legacy.bbt_ortho_mult_untied(th_d, x_d)
    check((y,) + grads(y, (th_d, x_d), dev(g)), lo.bbt_ortho_mult_untied(th, x, g), ("y", "d_theta", "d_x"))
    tht = rng.uniform(0, 2 * np.pi, (S, nblocks * 2, n - 1))
    tht_d = dev(tht).requires_grad_()
    y = legacy.bbt_ortho_mult_tied(tht_d, x_d)
    check((y,) + grads(y, (tht_d, x_d), dev(g)), lo.bbt_ortho_mult_tied(tht, x, g), ("y", "d_theta", "d_x"))
    say("legacy odo", n)
    diag = rng.uniform(0.1, 1.1, (S, nblocks, n))
    diag_d = dev(diag).requires_grad_()
    y = legacy.odo_mult_untied(th_d, diag_d, x_d)
    check((y,) + grads(y, (th_d, diag_d, x_d), dev(g)), lo.odo_mult_untied(th, diag, x, g),
          ("y", "d_theta", "d_diag", "d_x"))


def _module_reference(b, x):
    """The layer's forward restated with the oracle's functions and numpy pre / post processing
    (pad to n, one copy per stack; stacks side by side, summed over when they cover the padded
    output twice or more, first out_size columns, bias: butterfly/butterfly.py:193-276)."""
    p = {k: v.detach().cpu().numpy().astype(np.float64) for k, v in b.named_parameters()}
    n, S = b.in_size_extended, b.nstack
    cplx = b.complex
    if cplx:
        x = x[..., 0] + 1j * x[..., 1]
        for k in ("twiddle", "bias"):
            if k in p:
                p[k] = p[k][..., 0] + 1j * p[k][..., 1]
    xb = np.zeros((x.shape[0], n), dtype=x.dtype)
    xb[:, :b.in_size] = x
    xs = np.repeat(xb[:, None], S, axis=1)
    inc = b.increasing_stride
    if b.param == "regular":
        if b.tied_weight:
            y = lo.butterfly_mult(p["twiddle"], xs, inc)
        elif b.nblocks == 0:
            y = lo.butterfly_mult_untied_fast(p["twiddle"], xs, inc) if b.fast else lo.butterfly_mult_untied(p["twiddle"], xs, inc)
        else:
            y = lo.bbt_mult_untied_fast(p["twiddle"], xs) if b.fast else lo.bbt_mult_untied(p["twiddle"], xs)
    elif b.param == "ortho":
        if b.tied_weight:
            y = lo.butterfly_ortho_mult_tied(p["twiddle"], xs, inc)
        else:
            y = lo.butterfly_ortho_mult_untied(p["twiddle"], xs, inc) if b.nblocks == 0 else lo.bbt_ortho_mult_untied(p["twiddle"], xs)
    elif b.param == "odo" and b.fast:
        assert not b.tied_weight
        y = lo.odo_mult_untied(p["twiddle"], p["diag"], xs)
    elif b.param == "odo":
        if b.tied_weight:
            one = (lambda t, v, i: lo.butterfly_ortho_mult_tied(t, v, i)) if b.nblocks == 0 else (lambda t, v, i: lo.bbt_ortho_mult_tied(t, v))
            y = one(p["twiddle1"], one(p["twiddle"], xs, False) * p["diag"], True)
        else:
            one = (lambda t, v, i: lo.butterfly_ortho_mult_untied(t, v, i)) if b.nblocks == 0 else (lambda t, v, i: lo.bbt_ortho_mult_untied(t, v))
            y = one(p["twiddle1"], one(p["twiddle"], xs, inc) * p["diag"], not inc)
    else:
        raise AssertionError(b.param)
    flat = y.reshape(x.shape[0], S * n)
    out_ext = 1 << int(math.ceil(math.log2(b.out_size)))
    if (S * n) // out_ext >= 2:
        flat = flat.reshape(x.shape[0], (S * n) // out_ext, out_ext).sum(axis=1)
    flat = flat[:, :b.out_size]
    if "bias" in p:
        flat = flat + p["bias"]
    return flat


def test_layer_configurations():
    """The grid of tests_old/test_butterfly.py:19-52 (shapes; unit-norm factors after
    ortho_init), plus the values against the oracle for the configurations it covers."""
    from butterfly_amd.legacy import Butterfly
    torch.manual_seed(0)
    batch = 10
    count = 0
    for (in_size, out_size), cplx, tied, inc, ortho_init in itertools.product(
            [(7, 15), (15, 7)], [False, True], [True, False], [True, False], [False, True]):
        for param in (["regular"] if cplx else ["regular", "ortho", "odo", "obdobt"]):
            for nblocks in (0, 1, 2, 3):
                for expansion in (1, 2):
                    if param == "obdobt" and tied:
                        continue
                    if nblocks > 0 and cplx:
                        continue
                    if nblocks > 0 and not (tied and param == "odo") and tied:
                        continue
                    for fast in (True, False):
                        if param == "odo" and fast and nblocks == 0:
                            with pytest.raises(ValueError):
                                Butterfly(in_size, out_size, True, cplx, tied, inc, ortho_init, param,
                                          nblocks=nblocks, expansion=expansion, fast=fast)
                            continue
                        b = Butterfly(in_size, out_size, True, cplx, tied, inc, ortho_init, param,
                                      nblocks=nblocks, expansion=expansion, fast=fast).cuda()
                        x = torch.randn((batch, in_size) + ((2,) if cplx else ()), device="cuda")
                        y = b(x)
                        count += 1
                        assert y.shape == (batch, out_size) + ((2,) if cplx else ()), (y.shape, b)
                        if ortho_init and param == "regular" and not b.fast:
                            t = b.twiddle.detach().cpu().numpy()
                            t = (t[..., 0] + 1j * t[..., 1]) if cplx else t
                            assert np.allclose(np.linalg.norm(t.reshape(-1, 2, 2), ord=2, axis=(1, 2)), 1, atol=1e-5)
                        if param != "obdobt" and not (param == "odo" and b.fast and tied):
                            ref = _module_reference(b, x.cpu().numpy().astype(np.float64))
                            got = y.detach().cpu().numpy()
                            got = got[..., 0] + 1j * got[..., 1] if cplx else got
                            assert rel_err(got, ref) < 2e-5, (rel_err(got, ref), b)
    say("legacy layer configurations run:", count)
    assert count > 300


def test_layer_expansion_is_a_sum_of_butterflies():
    """tests_old/test_butterfly.py:54-69."""
    from butterfly_amd.legacy import Butterfly, butterfly_ortho_mult_tied
    torch.manual_seed(1)
    b = Butterfly(16, 16, bias=False, tied_weight=True, param="odo", expansion=4, diag_init="normal", fast=False).cuda()
    x = torch.randn(1, 16, device="cuda")
    total = 0
    for i in range(4):
        t = butterfly_ortho_mult_tied(b.twiddle[[i]], x.unsqueeze(1), False)
        t = t * b.diag[i]
        total = total + butterfly_ortho_mult_tied(b.twiddle1[[i]], t, True)
    assert torch.allclose(b(x), total.reshape(1, 16), atol=1e-5)


def test_bmm_layer_equals_a_loop_over_layers():
    """tests_old/test_butterfly.py:72-116."""
    from butterfly_amd.legacy import Butterfly, ButterflyBmm
    torch.manual_seed(2)
    batch, mb = 10, 3
    for (in_size, out_size), cplx, tied, inc, expansion in itertools.product(
            [(7, 15), (15, 7)], [False, True], [True, False], [True, False], [1, 2]):
        bmm = ButterflyBmm(in_size, out_size, mb, True, cplx, tied, inc, expansion=expansion).cuda()
        x = torch.randn((batch, mb, in_size) + ((2,) if cplx else ()), device="cuda")
        y = bmm(x)
        assert y.shape == (batch, mb, out_size) + ((2,) if cplx else ())
        loop = []
        for i in range(mb):
            b = Butterfly(in_size, out_size, True, cplx, tied, inc, expansion=expansion).cuda()
            b.twiddle = torch.nn.Parameter(bmm.twiddle[i * bmm.nstack:(i + 1) * bmm.nstack])
            b.bias = torch.nn.Parameter(bmm.bias[i])
            loop.append(b(x[:, i]))
        assert torch.allclose(y, torch.stack(loop, dim=1), atol=1e-5)
    # gradients reach every parameter
    bmm = ButterflyBmm(16, 16, mb, True, False, False, param="odo", nblocks=2).cuda()
    bmm(torch.randn(batch, mb, 16, device="cuda")).square().sum().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in bmm.parameters())


def im2col(x, k, pad):
    """(b, c, h, w) -> patches (b * h_out * w_out, k * k, c): the input channels under every
    kernel position of every output pixel, by explicit loops; and the index bookkeeping that
    lets the adjoint be formed the same way."""
    b, c, h, w = x.shape
    xp = np.zeros((b, c, h + 2 * pad, w + 2 * pad), x.dtype)
    xp[:, :, pad:pad + h, pad:pad + w] = x
    ho, wo = h + 2 * pad - (k - 1), w + 2 * pad - (k - 1)
    out = np.zeros((b, ho, wo, k * k, c), x.dtype)
    for i in range(k):
        for j in range(k):
            out[:, :, :, i * k + j, :] = xp[:, :, i:i + ho, j:j + wo].transpose(0, 2, 3, 1)
    return out.reshape(b * ho * wo, k * k, c)


def col2im(dp, shape, k, pad):
    """Adjoint of im2col: patch gradients (b * h_out * w_out, k * k, c) summed back onto the image."""
    b, c, h, w = shape
    ho, wo = h + 2 * pad - (k - 1), w + 2 * pad - (k - 1)
    dp = dp.reshape(b, ho, wo, k * k, c)
    dxp = np.zeros((b, c, h + 2 * pad, w + 2 * pad), dp.dtype)
    for i in range(k):
        for j in range(k):
            dxp[:, :, i:i + ho, j:j + wo] += dp[:, :, :, i * k + j, :].transpose(0, 3, 1, 2)
    return dxp[:, :, pad:pad + h, pad:pad + w]


@pytest.mark.parametrize("c,h,w,k,pad,copies", [(8, 5, 6, 3, 1, 1), (16, 4, 4, 3, 0, 2), (4, 7, 3, 1, 0, 3), (32, 6, 6, 5, 2, 1)])
def test_conv2d_multiplies(c, h, w, k, pad, copies):
    """butterfly_mult_conv2d / bbt_mult_conv2d: every kernel position's patch through its own
    butterflies, against explicit patch extraction + the numpy restatement, with the gradient
    of the image formed by the explicit adjoint of the patch extraction."""
    from butterfly_amd import legacy
    m = c.bit_length() - 1
    rng = np.random.default_rng(700 + c + k)
    b = 3
    S = k * k * copies
    x = rnd(rng, (b, c, h, w))
    patches = np.repeat(im2col(x, k, pad)[:, :, None, :], copies, axis=2).reshape(-1, S, c)
    g = rnd(rng, patches.shape)
    back = lambda t: t.detach().cpu().numpy().astype(np.float64)
    for inc in (True, False):
        say("conv2d multiply", c, h, w, k, pad, copies, inc)
        tw = rnd(rng, (S, m, c // 2, 2, 2)) / math.sqrt(2)
        y_ref, dtw_ref, dp_ref = lo.butterfly_mult_untied(tw, patches, inc, g)
        dx_ref = col2im(dp_ref.reshape(-1, k * k, copies, c).sum(axis=2), x.shape, k, pad)
        tw_d, x_d = dev(tw).requires_grad_(), dev(x).requires_grad_()
        y = legacy.butterfly_mult_conv2d(tw_d, x_d, k, pad, inc)
        dtw, dx = grads(y, (tw_d, x_d), dev(g))
        assert rel_err(back(y), y_ref) < FW_TOL
        assert rel_err(back(dx), dx_ref) < BW_TOL and rel_err(back(dtw), dtw_ref) < BW_TOL
    say("bbt conv2d", c, h, w, k, pad, copies)
    tw = rnd(rng, (S, 2 * 2 * m, c // 2, 2, 2)) / math.sqrt(2)
    y_ref, dtw_ref, dp_ref = lo.bbt_mult_untied(tw, patches, g)
    dx_ref = col2im(dp_ref.reshape(-1, k * k, copies, c).sum(axis=2), x.shape, k, pad)
    tw_d, x_d = dev(tw).requires_grad_(), dev(x).requires_grad_()
    y = legacy.bbt_mult_conv2d(tw_d, x_d, k, pad)
    dtw, dx = grads(y, (tw_d, x_d), dev(g))
    assert rel_err(back(y), y_ref) < FW_TOL
    assert rel_err(back(dx), dx_ref) < BW_TOL and rel_err(back(dtw), dtw_ref) < BW_TOL
    # a 1 x 1 kernel with one copy is the plain untied multiply over the pixels
    if k == 1 and copies == 1:
        flat = dev(x).permute(0, 2, 3, 1).reshape(-1, 1, c)
        assert torch.allclose(legacy.butterfly_mult_conv2d(tw_d[:, :m], dev(x), 1, 0, True),
                              legacy.butterfly_mult_untied(tw_d[:, :m], flat, True))


@pytest.mark.parametrize("n,cplx", [(2, False), (16, True), (64, False)])
def test_mult_factors(n, cplx):
    """butterfly_mult_factors: the tied product without a stack dimension, and its stack of
    intermediate values factor by factor."""
    from butterfly_amd import legacy
    m = n.bit_length() - 1
    rng = np.random.default_rng(800 + n)
    x, g = rnd(rng, (7, n), cplx), rnd(rng, (7, n), cplx)
    to_dev, back = (pairs, unpairs) if cplx else (dev, lambda t: t.detach().cpu().numpy().astype(np.float64))
    for inc in (True, False):
        say("mult_factors", n, cplx, inc)
        tied = rnd(rng, (n - 1, 2, 2), cplx) / math.sqrt(2)
        y_ref, dtw_ref, dx_ref = lo.butterfly_mult(tied[None], x[:, None], inc, g[:, None])
        tw_d, x_d = to_dev(tied).requires_grad_(), to_dev(x).requires_grad_()
        y = legacy.butterfly_mult_factors(tw_d, x_d, inc)
        dtw, dx = grads(y, (tw_d, x_d), to_dev(g))
        assert rel_err(back(y), y_ref[:, 0]) < FW_TOL
        assert rel_err(back(dx), dx_ref[:, 0]) < BW_TOL and rel_err(back(dtw), dtw_ref[0]) < BW_TOL
        steps = legacy.butterfly_mult_factors(tw_d, x_d, inc, return_intermediates=True)
        assert steps.shape[0] == m + 1
        value = x[:, None]
        assert rel_err(back(steps[0]), value[:, 0]) < FW_TOL
        for i, log_stride in enumerate(range(m) if inc else range(m - 1, -1, -1)):
            value = lo.factor_apply(lo.tied_expand(tied[None], log_stride, n), log_stride, value)
            assert rel_err(back(steps[i + 1]), value[:, 0]) < FW_TOL
        assert rel_err(back(steps[-1]), y_ref[:, 0]) < FW_TOL


def test_learnable_permutation_on_the_device():
    """The relaxed permutation product is plain tensor work: on the device it gives what it
    gives on the host (which tests/test_host.py holds against dense matrices), gradients included."""
    from butterfly_amd import legacy_permutation as lp
    torch.manual_seed(11)
    for n, share, inc, tail in [(64, False, False, ()), (256, True, True, (2,)), (1024, False, True, ())]:
        say("learnable permutation", n, share, inc, tail)
        host = lp.Permutation(n, share_logit=share, increasing_stride=inc).double()
        onboard = lp.Permutation(n, share_logit=share, increasing_stride=inc).double().cuda()
        with torch.no_grad():
            onboard.logit.copy_(host.logit)
        x = torch.randn(33, n, *tail, dtype=torch.float64)
        g = torch.randn(33, n, *tail, dtype=torch.float64)
        xh, xd = x.clone().requires_grad_(), x.cuda().requires_grad_()
        yh, yd = host(xh), onboard(xd)
        gh = torch.autograd.grad(yh, (xh, host.logit), g)
        gd = torch.autograd.grad(yd, (xd, onboard.logit), g.cuda())
        assert torch.allclose(yd.cpu(), yh, atol=1e-12)
        for a, b in zip(gd, gh):
            assert torch.allclose(a.cpu(), b, atol=1e-10)
        assert onboard.argmax().cpu().tolist() == host.argmax().tolist()
