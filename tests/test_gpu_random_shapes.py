"""Seeded sweep over randomly drawn problems: dtype, base, log_n, blocks, stacks, batch (ragged
against every row-group size), padded / trimmed widths, stride order, operand strides (dense,
every other element, a stack broadcast with stride 0, rows with a gap), plain backward or the
forward that keeps activations.  Every case through the C ABI against the CPU oracle:
max|err| / max|ref| <= 1e-5 forward, <= 1e-4 gradients.  The draw is fixed by the seed, so the
cases are the same in every run; each is printed before it starts."""
import sys

import numpy as np
import pytest
import torch

from conftest import randn, rel_err
from oracle import oracle

pytestmark = pytest.mark.gpu

FW_TOL = 1e-5
BW_TOL = 1e-4
BUDGET = 1 << 23        # batch * stacks * n * stages per case: keeps the scalar oracle at a fraction of a second


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def draw_case(rng, base4):
    dtype = np.complex64 if rng.random() < 0.3 else np.float32
    L = int(rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 10, 11, 12, 13]))
    if base4 and L < 2:
        L = 2
    n = 1 << L
    nb = int(rng.choice([1, 1, 2, 2, 3, 4]))
    S = int(rng.choice([1, 1, 2, 3]))
    max_b = max(1, BUDGET // (S * n * nb * L))
    B = int(min(max_b, rng.choice([1, 2, 3, 5, 17, 64, 129, 300, 1000, 2049, 5000])))
    kind_i = rng.choice(["full", "short", "long"], p=[0.6, 0.3, 0.1])
    I = n if kind_i == "full" else (int(rng.integers(1, n + 1)) if kind_i == "short" else n + int(rng.integers(1, 40)))
    O = n if rng.random() < 0.6 else int(rng.integers(1, n + 1))
    inc = bool(rng.random() < 0.5)
    layout = str(rng.choice(["dense", "every-other", "broadcast", "gap"]))
    return dtype, B, S, L, nb, I, O, inc, layout


def strided_input(rng, dtype, B, S, I, layout):
    """(host array, device tensor) of shape (B, S, I) whose device strides follow `layout`."""
    if layout == "every-other":
        full = torch.from_numpy(randn(rng, (B, S, 2 * I), dtype)).cuda()
        xd = full[:, :, ::2]
    elif layout == "broadcast" and S > 1:
        full = torch.from_numpy(randn(rng, (B, 1, I), dtype)).cuda()
        xd = full.expand(B, S, I)
    elif layout == "gap":
        full = torch.from_numpy(randn(rng, (B, S, I + 5), dtype)).cuda()
        xd = full[:, :, :I]
    else:
        xd = torch.from_numpy(randn(rng, (B, S, I), dtype)).cuda()
    return np.ascontiguousarray(xd.cpu().numpy()), xd


@pytest.mark.parametrize("chunk", range(4))
def test_random_base2_problems(chunk):
    from butterfly_amd import _capi
    rng = np.random.default_rng(9100 + chunk)
    for i in range(30):
        dtype, B, S, L, nb, I, O, inc, layout = draw_case(rng, False)
        n = 1 << L
        saving = bool(rng.random() < 0.4)
        say(f"random base-2 case {chunk}.{i}:", np.dtype(dtype).name, (B, S, L, nb, I, O, inc, layout), "saving" if saving else "")
        tw = (randn(rng, (S, nb, L, n // 2, 2, 2), dtype) / np.sqrt(2)).astype(dtype)
        x, xd = strided_input(rng, dtype, B, S, I, layout)
        g = randn(rng, (B, S, O), dtype)
        twd, gd = torch.from_numpy(tw).cuda(), torch.from_numpy(g).cuda()
        y_ref = oracle.butterfly_fw(tw, x, inc, O)
        dtw_ref, dx_ref = oracle.butterfly_bw(tw, x, g, inc)
        res = _capi.multiply_fw_bw_saving(twd, xd, gd, inc, O) if saving else None
        if res is not None:
            y, dtw, dx, _ = res
        else:
            y = _capi.multiply_fw(twd, xd, inc, O)
            dtw, dx = _capi.multiply_bw(twd, xd, gd, inc)
        torch.cuda.synchronize()
        assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL
        assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
        assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL


@pytest.mark.parametrize("chunk", range(2))
def test_random_base4_problems(chunk):
    from butterfly_amd import _capi
    rng = np.random.default_rng(9200 + chunk)
    for i in range(30):
        dtype, B, S, L, nb, I, O, inc, layout = draw_case(rng, True)
        n = 1 << L
        saving = bool(rng.random() < 0.4)
        say(f"random base-4 case {chunk}.{i}:", np.dtype(dtype).name, (B, S, L, nb, I, O, inc, layout), "saving" if saving else "")
        tw4 = (randn(rng, (S, nb, L // 2, n // 4, 4, 4), dtype) / 2).astype(dtype)
        tw2 = (randn(rng, (S, nb, L % 2, n // 2, 2, 2), dtype) / np.sqrt(2)).astype(dtype)
        x, xd = strided_input(rng, dtype, B, S, I, layout)
        g = randn(rng, (B, S, O), dtype)
        t4, t2, gd = torch.from_numpy(tw4).cuda(), torch.from_numpy(tw2).cuda(), torch.from_numpy(g).cuda()
        y_ref = oracle.butterfly_base4_fw(tw4, tw2, x, inc, O)
        d4_ref, d2_ref, dx_ref = oracle.butterfly_base4_bw(tw4, tw2, x, g, inc)
        res = _capi.multiply_base4_fw_bw_saving(t4, t2, xd, gd, inc, O) if saving else None
        if res is not None:
            y, d4, d2, dx = res
        else:
            y = _capi.multiply_base4_fw(t4, t2, xd, inc, O)
            d4, d2, dx = _capi.multiply_base4_bw(t4, t2, xd, gd, inc)
        torch.cuda.synchronize()
        assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL
        assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
        assert rel_err(d4.cpu().numpy(), d4_ref) < BW_TOL
        if L % 2:
            assert rel_err(d2.cpu().numpy(), d2_ref) < BW_TOL


@pytest.mark.parametrize("chunk", range(2))
def test_random_fused_operator_problems(chunk):
    """The operator that takes column tables and a bias, under autograd, against the same
    computation spelled out with PyTorch gathers and adds around `butterfly_multiply` (which the
    sweeps above hold against the oracle): output and every gradient."""
    import butterfly_amd  # noqa: F401
    ops = torch.ops.torch_butterfly
    rng = np.random.default_rng(9300 + chunk)
    torch.manual_seed(9300 + chunk)
    for i in range(25):
        dtype, B, S, L, nb, I, O, inc, _ = draw_case(rng, False)
        n = 1 << L
        I = min(I, n)
        which = str(rng.choice(["io", "i", "o"]))
        with_bias = bool(rng.random() < 0.5)
        say(f"random fused case {chunk}.{i}:", np.dtype(dtype).name, (B, S, L, nb, I, O, inc, which, with_bias))
        tdt = torch.complex64 if np.dtype(dtype).kind == "c" else torch.float32
        tw = (torch.randn(S, nb, L, n // 2, 2, 2, dtype=tdt) / 2 ** 0.5).cuda().requires_grad_()
        x = torch.randn(B, S, I, dtype=tdt).cuda().requires_grad_()
        bias = torch.randn(S, O, dtype=tdt).cuda().requires_grad_() if with_bias else None
        g = torch.randn(B, S, O, dtype=tdt).cuda()
        p_in = torch.cat((torch.randperm(I), torch.arange(I, n))).cuda()
        q = torch.randperm(O).cuda()
        full_q = torch.cat((q, torch.arange(O, n).cuda()))
        out_index = torch.empty_like(full_q)
        out_index[full_q] = torch.arange(n).cuda()
        t_in = p_in.int() if "i" in which else None
        t_out = out_index.int() if "o" in which else None
        y = ops.butterfly_multiply_perm(tw, x, t_in, t_out, bias, inc, O)
        wrt = (tw, x) + ((bias,) if with_bias else ())
        got = torch.autograd.grad(y, wrt, g)
        u = torch.nn.functional.pad(x, (0, n - I))
        if "i" in which:
            u = u[..., p_in]
        y2 = ops.butterfly_multiply(tw, u, inc, O)
        if with_bias:
            y2 = y2 + bias
        if "o" in which:
            y2 = y2[..., q]
        want = torch.autograd.grad(y2, wrt, g)
        torch.cuda.synchronize()
        for a, b in [(y, y2)] + list(zip(got, want)):
            assert a.shape == b.shape
            assert (a - b).abs().max().item() <= BW_TOL * max(1.0, b.abs().max().item())
