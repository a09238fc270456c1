"""Parity of the HIP library (through its C ABI and through the registered operators)
against the CPU oracle.  Tolerances are max|err| / max|ref|: 1e-5 forward, 1e-4 gradients."""
import ctypes
import sys

import numpy as np
import pytest
import torch

from conftest import randn, rel_err
from oracle import oracle

pytestmark = pytest.mark.gpu

FW_TOL = 1e-5
BW_TOL = 1e-4


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def make_case(rng, dtype, B, S, L, nb, I=None, O=None):
    n = 1 << L
    I = n if I is None else I
    tw = (randn(rng, (S, nb, L, n // 2, 2, 2), dtype) / np.sqrt(2)).astype(dtype)
    x = randn(rng, (B, S, I), dtype)
    g = randn(rng, (B, S, n if O is None else O), dtype)
    return tw, x, g


CASES = [
    # dtype, B, S, L, nb, I, O, inc
    (np.float32, 7, 1, 1, 1, None, None, True),
    (np.float32, 5, 2, 2, 3, None, None, False),
    (np.float32, 33, 2, 5, 3, 15, None, True),
    (np.float32, 10, 2, 5, 3, 28, 14, False),
    (np.float32, 10, 2, 5, 2, 71, 27, True),
    (np.float32, 64, 1, 10, 1, None, None, True),
    (np.float32, 50, 1, 10, 2, None, None, False),
    (np.float32, 10, 2, 12, 3, None, None, True),
    (np.float32, 10, 2, 12, 3, 4092, 2046, False),
    (np.float32, 3, 1, 14, 1, None, None, False),
    (np.complex64, 9, 2, 3, 2, None, None, True),
    (np.complex64, 10, 2, 5, 3, 2 * 32 + 7, 32 - 5, False),
    (np.complex64, 40, 1, 9, 2, None, None, False),
    (np.complex64, 10, 2, 12, 3, None, None, True),
    (np.complex64, 6, 1, 12, 1, 2047, None, False),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{np.dtype(c[0]).name}-B{c[1]}-S{c[2]}-L{c[3]}-nb{c[4]}-I{c[5]}-O{c[6]}-inc{int(c[7])}")
def test_c_abi_matches_oracle(case):
    from butterfly_amd import _capi
    dtype, B, S, L, nb, I, O, inc = case
    say("case", case)
    rng = np.random.default_rng(hash((L, nb, B, S)) % (1 << 31))
    tw, x, g = make_case(rng, dtype, B, S, L, nb, I, O)
    y_ref = oracle.butterfly_fw(tw, x, inc, O)
    dtw_ref, dx_ref = oracle.butterfly_bw(tw, x, g, inc)
    y = _capi.multiply_fw(dev(tw), dev(x), inc, O)
    dtw, dx = _capi.multiply_bw(dev(tw), dev(x), dev(g), inc)
    torch.cuda.synchronize()
    assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL


@pytest.mark.parametrize("L", list(range(1, 11)))
def test_register_resident_kernels_all_sizes(L):
    """n = 2 .. 1024 with one or two blocks run on the twiddle-stationary kernels: every
    size, both stride orders, ragged batch (partial row groups), padded input, sliced
    output, two stacks."""
    from butterfly_amd import _capi
    n = 1 << L
    rng = np.random.default_rng(500 + L)
    for nb in (1, 2):
        for inc in (True, False):
            for B, S, I, O in [(1, 1, n, n), (37, 2, n, n), (300, 1, max(1, n - 1), max(1, n - 1)),
                               (19, 2, n + 5, max(1, n // 2))]:
                say("fast case", L, nb, inc, B, S, I, O)
                tw, x, g = make_case(rng, np.float32, B, S, L, nb, I, O)
                y_ref = oracle.butterfly_fw(tw, x, inc, O)
                dtw_ref, dx_ref = oracle.butterfly_bw(tw, x, g, inc)
                y = _capi.multiply_fw(dev(tw), dev(x), inc, O)
                dtw, dx = _capi.multiply_bw(dev(tw), dev(x), dev(g), inc)
                torch.cuda.synchronize()
                assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL, (L, nb, inc, B, S, I, O)
                assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL, (L, nb, inc, B, S, I, O)
                assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL, (L, nb, inc, B, S, I, O)


MULTIPASS_CASES = [
    # B, S, L, nb, I, O, inc -- more than two blocks and rows of 2048 / 4096 (chunk + span passes)
    (40, 2, 9, 3, None, None, True),
    (40, 2, 9, 4, None, None, False),
    (33, 1, 10, 5, 1000, 900, False),
    (21, 2, 11, 1, None, None, True),
    (21, 2, 11, 1, None, None, False),
    (21, 1, 11, 2, None, None, True),
    (21, 1, 11, 2, 2000, 1500, False),
    (13, 2, 12, 1, None, None, True),
    (13, 2, 12, 1, None, None, False),
    (13, 1, 12, 2, None, None, True),
    (13, 1, 12, 2, None, None, False),
    (10, 2, 12, 3, 4092, 2046, True),
    (10, 2, 12, 3, 2 * 4096 + 7, 4091, False),
    (300, 1, 12, 2, None, None, True),
    # many rows per workgroup: the row slots in LDS and the transpose buffers go round several times
    (3000, 1, 10, 2, None, None, False),
    (5000, 1, 10, 1, None, None, True),
    (4500, 1, 10, 1, 1000, 1024, False),
    (4400, 2, 8, 1, None, 200, True),
    (9000, 1, 7, 2, 100, 120, True),
    (1500, 1, 12, 1, None, None, True),
    (1500, 1, 12, 1, None, None, False),
    (1300, 2, 11, 2, 2000, 2040, False),
]


@pytest.mark.parametrize("case", MULTIPASS_CASES, ids=lambda c: f"B{c[0]}-S{c[1]}-L{c[2]}-nb{c[3]}-I{c[4]}-O{c[5]}-inc{int(c[6])}")
def test_multi_launch_schedules(case):
    from butterfly_amd import _capi
    B, S, L, nb, I, O, inc = case
    say("multipass case", case)
    rng = np.random.default_rng(900 + L * 13 + nb)
    tw, x, g = make_case(rng, np.float32, B, S, L, nb, I, O)
    y_ref = oracle.butterfly_fw(tw, x, inc, O)
    dtw_ref, dx_ref = oracle.butterfly_bw(tw, x, g, inc)
    y = _capi.multiply_fw(dev(tw), dev(x), inc, O)
    dtw, dx = _capi.multiply_bw(dev(tw), dev(x), dev(g), inc)
    torch.cuda.synchronize()
    assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL


LONG_ROW_CASES = [
    # dtype, B, S, L, nb, I, O, inc -- rows beyond 4096: chunk passes for bits 0..9 and one span
    # pass per group of up to five higher bits (one and two spans, the block boundary inside the
    # top span, several row partitions)
    (np.float32, 9, 1, 13, 1, None, None, True),
    (np.float32, 9, 2, 13, 2, None, None, False),
    (np.float32, 7, 1, 14, 2, 16000, 9000, True),
    (np.float32, 5, 1, 15, 3, None, None, False),
    (np.float32, 3, 1, 16, 1, None, None, True),
    (np.float32, 2, 1, 17, 1, None, 70000, False),
    (np.float32, 300, 1, 13, 1, None, None, True),
    (np.complex64, 6, 1, 13, 2, None, None, True),
    (np.complex64, 4, 2, 14, 1, 9000, None, False),
    (np.complex64, 3, 1, 15, 1, None, None, True),
    (np.complex64, 120, 1, 13, 1, None, None, False),
]


@pytest.mark.parametrize("case", LONG_ROW_CASES, ids=lambda c: f"{np.dtype(c[0]).name}-B{c[1]}-S{c[2]}-L{c[3]}-nb{c[4]}-I{c[5]}-O{c[6]}-inc{int(c[7])}")
def test_long_rows(case):
    from butterfly_amd import _capi
    dtype, B, S, L, nb, I, O, inc = case
    say("long-row case", case)
    rng = np.random.default_rng(1900 + L * 13 + nb)
    tw, x, g = make_case(rng, dtype, B, S, L, nb, I, O)
    y_ref = oracle.butterfly_fw(tw, x, inc, O)
    dtw_ref, dx_ref = oracle.butterfly_bw(tw, x, g, inc)
    y = _capi.multiply_fw(dev(tw), dev(x), inc, O)
    dtw, dx = _capi.multiply_bw(dev(tw), dev(x), dev(g), inc)
    torch.cuda.synchronize()
    assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL


def test_operands_beyond_two_gib():
    """Operands of 3 GiB: workgroups address rows with 32-bit offsets from their first row, so
    the host gives each one few enough rows.  Forward and d_input rows against the oracle on a
    sample of rows; d_twiddle against the sum of two half-batch calls (each below 2 GiB)."""
    from butterfly_amd import _capi
    L, B = 16, 12288
    n = 1 << L
    say("big operands", L, B)
    torch.manual_seed(77)
    tw = (torch.randn(1, 1, L, n // 2, 2, 2) / 2 ** 0.5).cuda()
    x = torch.randn(B, 1, n, device="cuda")
    g = torch.randn(B, 1, n, device="cuda")
    y = _capi.multiply_fw(tw, x, True)
    dtw, dx = _capi.multiply_bw(tw, x, g, True)
    torch.cuda.synchronize()
    rows = [0, 1, 47, 48, 49, B // 2 - 1, B // 2, B - 2, B - 1] + list(range(6000, 6144, 16))
    twn = tw.cpu().numpy()
    xs, gs = x[rows].cpu().numpy(), g[rows].cpu().numpy()
    y_ref = oracle.butterfly_fw(twn, xs, True)
    _, dx_ref = oracle.butterfly_bw(twn, xs, gs, True)
    assert rel_err(y[rows].cpu().numpy(), y_ref) < FW_TOL
    assert rel_err(dx[rows].cpu().numpy(), dx_ref) < BW_TOL
    h = B // 2
    d1, dxa = _capi.multiply_bw(tw, x[:h], g[:h], True)
    d2, dxb = _capi.multiply_bw(tw, x[h:], g[h:], True)
    torch.cuda.synchronize()
    assert torch.equal(dxa, dx[:h]) and torch.equal(dxb, dx[h:])
    ref = (d1.double() + d2.double())
    assert ((dtw.double() - ref).abs().max() / ref.abs().max()).item() < BW_TOL


WIDE_CASES = [
    # dtype, B, S, L, nb, I, O, inc -- enough rows for the whole-block forward kernel (the host
    # picks it from a row count on; below that the chunked passes run)
    (np.float32, 2100, 1, 12, 1, None, None, True),
    (np.float32, 1050, 2, 12, 1, 4000, 4090, False),
    (np.float32, 8200, 1, 12, 2, None, None, True),
    (np.float32, 4100, 1, 11, 2, None, 2047, False),
    (np.float32, 3, 1, 11, 1, None, None, True),
    (np.complex64, 260, 1, 11, 1, None, None, True),
    (np.complex64, 1030, 2, 11, 2, 2000, None, False),
]


@pytest.mark.parametrize("case", WIDE_CASES, ids=lambda c: f"{np.dtype(c[0]).name}-B{c[1]}-S{c[2]}-L{c[3]}-nb{c[4]}-I{c[5]}-O{c[6]}-inc{int(c[7])}")
def test_whole_block_forward_kernel(case):
    from butterfly_amd import _capi
    dtype, B, S, L, nb, I, O, inc = case
    say("wide case", case)
    plan = _capi.describe_plan(int(np.dtype(dtype).kind == "c"), B, S, L, nb, inc, False)
    assert all(line.startswith("wide") for line in plan), plan
    rng = np.random.default_rng(3100 + L * 13 + nb)
    tw, x, _ = make_case(rng, dtype, B, S, L, nb, I, O)
    y_ref = oracle.butterfly_fw(tw, x, inc, O)
    y = _capi.multiply_fw(dev(tw), dev(x), inc, O)
    torch.cuda.synchronize()
    assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL


COMPLEX_FAST_CASES = [
    # B, S, L, nb, I, O, inc
    (37, 2, 1, 2, None, None, True),
    (37, 2, 3, 3, None, None, False),
    (300, 1, 5, 2, 29, 20, True),
    (50, 2, 6, 1, None, None, False),
    (50, 2, 8, 2, None, None, True),
    (40, 1, 9, 3, None, None, False),
    (33, 2, 10, 1, None, None, True),
    (33, 1, 10, 2, 1000, 1001, False),
    (9, 2, 11, 2, None, None, True),
    (9, 1, 12, 1, None, None, True),
    (9, 1, 12, 2, None, None, False),
    (5, 2, 12, 3, 4092, 2046, True),
    (1400, 1, 10, 1, None, None, True),
    (700, 1, 11, 1, None, None, True),
    (700, 1, 11, 2, None, None, False),
]


@pytest.mark.parametrize("case", COMPLEX_FAST_CASES, ids=lambda c: f"B{c[0]}-S{c[1]}-L{c[2]}-nb{c[3]}-I{c[4]}-O{c[5]}-inc{int(c[6])}")
def test_complex_register_resident_kernels(case):
    from butterfly_amd import _capi
    B, S, L, nb, I, O, inc = case
    say("complex case", case)
    rng = np.random.default_rng(1300 + L * 17 + nb)
    tw, x, g = make_case(rng, np.complex64, B, S, L, nb, I, O)
    y_ref = oracle.butterfly_fw(tw, x, inc, O)
    dtw_ref, dx_ref = oracle.butterfly_bw(tw, x, g, inc)
    y = _capi.multiply_fw(dev(tw), dev(x), inc, O)
    dtw, dx = _capi.multiply_bw(dev(tw), dev(x), dev(g), inc)
    torch.cuda.synchronize()
    assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL


def test_c_abi_strided_operands():
    """Stride-0 stack broadcast (what Butterfly.pre_process hands over), a transposed input
    and a non-contiguous gradient."""
    from butterfly_amd import _capi
    rng = np.random.default_rng(11)
    B, S, L, nb = 12, 3, 6, 2
    n = 1 << L
    tw = (randn(rng, (S, nb, L, n // 2, 2, 2), np.float32) / np.sqrt(2)).astype(np.float32)
    x1 = randn(rng, (B, n), np.float32)
    x_np = np.broadcast_to(x1[:, None, :], (B, S, n))
    g_big = randn(rng, (B, S, 2 * n), np.float32)
    x_dev = dev(x1).unsqueeze(1).expand(B, S, n)
    g_dev = dev(g_big)[:, :, ::2]
    say("strided: expand + strided grad")
    y = _capi.multiply_fw(dev(tw), x_dev, True)
    dtw, dx = _capi.multiply_bw(dev(tw), x_dev, g_dev, True)
    y_ref = oracle.butterfly_fw(tw, x_np, True)
    dtw_ref, dx_ref = oracle.butterfly_bw(tw, x_np, g_big[:, :, ::2], True)
    assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL
    say("strided: transposed input")
    xt = dev(np.ascontiguousarray(x_np.transpose(2, 0, 1))).permute(1, 2, 0)
    assert not xt.is_contiguous()
    y2 = _capi.multiply_fw(dev(tw), xt, True)
    assert torch.equal(y2, y)


def _random_case(seed):
    rng = np.random.default_rng(seed)
    dtype = np.complex64 if rng.random() < 0.35 else np.float32
    L = int(rng.integers(1, 14))
    n = 1 << L
    nb = int(rng.integers(1, 4))
    S = int(rng.integers(1, 4))
    budget = (1 << 20) // (n * S * nb)                       # keeps the oracle to a fraction of a second
    B = int(rng.integers(1, max(2, min(400, budget + 1))))
    I = n if rng.random() < 0.4 else int(rng.integers(1, n + 6))
    O = None if rng.random() < 0.4 else int(rng.integers(1, n + 1))
    inc = bool(rng.integers(0, 2))
    layout = ["dense", "stack broadcast", "batch innermost", "padded rows"][int(rng.integers(0, 4))]
    return rng, dtype, B, S, L, nb, I, O, inc, layout


@pytest.mark.parametrize("seed", range(48))
def test_random_shapes_and_layouts(seed):
    """Seeded sweep over sizes, block counts, paddings, trims and input layouts through the C ABI."""
    from butterfly_amd import _capi
    rng, dtype, B, S, L, nb, I, O, inc, layout = _random_case(5000 + seed)
    say("random case", seed, np.dtype(dtype).name, B, S, L, nb, I, O, inc, layout)
    n = 1 << L
    tw = (randn(rng, (S, nb, L, n // 2, 2, 2), dtype) / np.sqrt(2)).astype(dtype)
    cols = n if O is None else O
    g = randn(rng, (B, S, cols), dtype)
    if layout == "stack broadcast":
        x1 = randn(rng, (B, I), dtype)
        x = np.ascontiguousarray(np.broadcast_to(x1[:, None, :], (B, S, I)))
        x_dev = dev(x1).unsqueeze(1).expand(B, S, I)
    elif layout == "batch innermost":
        x = randn(rng, (B, S, I), dtype)
        x_dev = dev(np.ascontiguousarray(x.transpose(1, 2, 0))).permute(2, 0, 1)
    elif layout == "padded rows":
        big = randn(rng, (B, S, I + 3), dtype)
        x = np.ascontiguousarray(big[:, :, :I])
        x_dev = dev(big)[:, :, :I]
    else:
        x = randn(rng, (B, S, I), dtype)
        x_dev = dev(x)
    y_ref = oracle.butterfly_fw(tw, x, inc, O)
    dtw_ref, dx_ref = oracle.butterfly_bw(tw, x, g, inc)
    y = _capi.multiply_fw(dev(tw), x_dev, inc, O)
    dtw, dx = _capi.multiply_bw(dev(tw), x_dev, dev(g), inc)
    torch.cuda.synchronize()
    assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL


BASE4_CASES = [
    (np.float32, 9, 2, 2, 1, None, None, True),
    (np.float32, 9, 2, 3, 2, None, None, False),
    (np.float32, 20, 4, 8, 1, None, None, True),
    (np.float32, 11, 2, 7, 3, 100, 90, False),
    (np.float32, 6, 1, 11, 2, None, None, True),
    (np.complex64, 7, 2, 5, 2, 40, 17, True),
    (np.complex64, 5, 1, 10, 2, None, None, False),
    (np.float32, 5, 2, 1, 2, None, None, True),
]


@pytest.mark.parametrize("case", BASE4_CASES, ids=lambda c: f"{np.dtype(c[0]).name}-B{c[1]}-S{c[2]}-L{c[3]}-nb{c[4]}-I{c[5]}-O{c[6]}-inc{int(c[7])}")
def test_c_abi_base4_matches_oracle(case):
    from butterfly_amd import _capi
    dtype, B, S, L, nb, I, O, inc = case
    say("base4 case", case)
    rng = np.random.default_rng(100 + L * 7 + nb)
    n = 1 << L
    I_ = n if I is None else I
    tw4 = (randn(rng, (S, nb, L // 2, n // 4, 4, 4), dtype) / 2).astype(dtype)
    tw2 = (randn(rng, (S, nb, L % 2, n // 2, 2, 2), dtype) / np.sqrt(2)).astype(dtype)
    x = randn(rng, (B, S, I_), dtype)
    g = randn(rng, (B, S, n if O is None else O), dtype)
    y_ref = oracle.butterfly_base4_fw(tw4, tw2, x, inc, O)
    d4_ref, d2_ref, dx_ref = oracle.butterfly_base4_bw(tw4, tw2, x, g, inc)
    y = _capi.multiply_base4_fw(dev(tw4), dev(tw2), dev(x), inc, O)
    d4, d2, dx = _capi.multiply_base4_bw(dev(tw4), dev(tw2), dev(x), dev(g), inc)
    assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(d4.cpu().numpy(), d4_ref) < BW_TOL
    assert rel_err(d2.cpu().numpy(), d2_ref) < BW_TOL


@pytest.mark.parametrize("L", [2, 4, 6, 8, 10])
def test_base4_register_resident_kernels(L):
    """Even log_n <= 10 in float runs on the base-4 twiddle-stationary kernels: every size,
    both stride orders, one to three blocks, ragged batch, padded input, sliced output."""
    from butterfly_amd import _capi
    n = 1 << L
    rng = np.random.default_rng(1700 + L)
    for nb in (1, 2, 3):
        for inc in (True, False):
            for B, S, I, O in [(1, 1, n, n), (37, 2, n, n), (300, 1, n - 1, n - 1), (19, 4, n + 5, n // 2)]:
                say("base4 fast case", L, nb, inc, B, S, I, O)
                tw4 = (randn(rng, (S, nb, L // 2, n // 4, 4, 4), np.float32) / 2).astype(np.float32)
                tw2 = np.zeros((S, nb, 0, n // 2, 2, 2), np.float32)
                x = randn(rng, (B, S, I), np.float32)
                g = randn(rng, (B, S, O), np.float32)
                y_ref = oracle.butterfly_base4_fw(tw4, tw2, x, inc, O)
                d4_ref, _, dx_ref = oracle.butterfly_base4_bw(tw4, tw2, x, g, inc)
                y = _capi.multiply_base4_fw(dev(tw4), dev(tw2), dev(x), inc, O)
                d4, _, dx = _capi.multiply_base4_bw(dev(tw4), dev(tw2), dev(x), dev(g), inc)
                torch.cuda.synchronize()
                assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL, (L, nb, inc, B, S, I, O)
                assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL, (L, nb, inc, B, S, I, O)
                assert rel_err(d4.cpu().numpy(), d4_ref) < BW_TOL, (L, nb, inc, B, S, I, O)


@pytest.mark.parametrize("dtype,L", [(np.float32, 3), (np.float32, 5), (np.float32, 7), (np.float32, 9)] +
                         [(np.complex64, L) for L in range(2, 9)],
                         ids=lambda v: np.dtype(v).name if isinstance(v, type) else str(v))
def test_base4_general_register_resident_kernels(dtype, L):
    """Odd log_n (the block ends with a 2x2 stage; bit pairs unaligned for decreasing stride) and
    complex64: every size, both stride orders, one to three blocks, ragged batch, padded input,
    sliced output, many row groups per workgroup."""
    from butterfly_amd import _capi
    n = 1 << L
    rng = np.random.default_rng(2700 + L)
    big = max(300, 5000 // (1 + (n > 64)))
    for nb in (1, 2, 3):
        for inc in (True, False):
            for B, S, I, O in [(1, 1, n, n), (37, 2, n, n), (big, 1, n - 1, n - 1), (19, 4, n + 5, max(1, n // 2))]:
                say("base4 general case", np.dtype(dtype).name, L, nb, inc, B, S, I, O)
                tw4 = (randn(rng, (S, nb, L // 2, n // 4, 4, 4), dtype) / 2).astype(dtype)
                tw2 = (randn(rng, (S, nb, L % 2, n // 2, 2, 2), dtype) / np.sqrt(2)).astype(dtype)
                x = randn(rng, (B, S, I), dtype)
                g = randn(rng, (B, S, O), dtype)
                y_ref = oracle.butterfly_base4_fw(tw4, tw2, x, inc, O)
                d4_ref, d2_ref, dx_ref = oracle.butterfly_base4_bw(tw4, tw2, x, g, inc)
                y = _capi.multiply_base4_fw(dev(tw4), dev(tw2), dev(x), inc, O)
                d4, d2, dx = _capi.multiply_base4_bw(dev(tw4), dev(tw2), dev(x), dev(g), inc)
                torch.cuda.synchronize()
                key = (L, nb, inc, B, S, I, O)
                assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL, key
                assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL, key
                assert rel_err(d4.cpu().numpy(), d4_ref) < BW_TOL, key
                if L % 2:
                    assert rel_err(d2.cpu().numpy(), d2_ref) < BW_TOL, key


def test_operators_match_oracle_and_autograd():
    """torch.ops.torch_butterfly.* end to end: views returned, autograd wired, lazy conj
    and transposed twiddle views accepted."""
    import butterfly_amd  # noqa: F401  (registers the operators)
    rng = np.random.default_rng(21)
    for dtype in (np.float32, np.complex64):
        B, S, L, nb, I, O = 6, 2, 5, 3, 29, 20
        n = 1 << L
        tw, x, g = make_case(rng, dtype, B, S, L, nb, I, O)
        say("ops", np.dtype(dtype).name)
        twd = dev(tw).requires_grad_()
        xd = dev(x).requires_grad_()
        y = torch.ops.torch_butterfly.butterfly_multiply(twd, xd, False, O)
        assert y.shape == (B, S, O) and y.stride() == (S * n, n, 1)   # a view of an n-wide buffer
        dtw, dx = torch.autograd.grad(y, (twd, xd), dev(g))
        y_ref = oracle.butterfly_fw(tw, x, False, O)
        dtw_ref, dx_ref = oracle.butterfly_bw(tw, x, g, False)
        assert rel_err(y.detach().cpu().numpy(), y_ref) < FW_TOL
        assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
        assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL
        # transposed + flipped (+ conjugated) twiddle view, as Butterfly.forward(transpose=True) builds
        tv = dev(tw).transpose(-1, -2).flip([1, 2])
        tv_np = np.ascontiguousarray(np.flip(np.swapaxes(tw, -1, -2), (1, 2)))
        if np.dtype(dtype).kind == "c":
            tv, tv_np = tv.conj(), tv_np.conj()
        y2 = torch.ops.torch_butterfly.butterfly_multiply_fw(tv, dev(x), True, None)
        assert rel_err(y2.cpu().numpy(), oracle.butterfly_fw(tv_np, x, True)) < FW_TOL


@pytest.mark.parametrize("L,nb", [(3, 1), (10, 2), (12, 2), (14, 1)])
def test_empty_batch(L, nb):
    """No rows at all: outputs and input gradients are empty tensors of the right shape, every
    d_twiddle (and d_bias) entry is an empty sum, i.e. exactly zero -- for every kernel family the
    size would otherwise pick, float and complex64, base 2, base 4, with bias and column tables."""
    import butterfly_amd  # noqa: F401
    ops = torch.ops.torch_butterfly
    n = 1 << L
    S, O = 2, n - 3
    for tdt in (torch.float32, torch.complex64):
        say("empty batch", L, nb, tdt)
        # scratch the allocator's blocks so that an output nobody writes does not read as zero
        junk = torch.full((S * nb * L * n * 8,), 7.0, device="cuda")
        del junk
        tw = torch.randn(S, nb, L, n // 2, 2, 2, dtype=tdt, device="cuda", requires_grad=True)
        x = torch.empty(0, S, n, dtype=tdt, device="cuda", requires_grad=True)
        g = torch.empty(0, S, O, dtype=tdt, device="cuda")
        y = ops.butterfly_multiply_fw(tw, x, True, O)
        assert y.shape == (0, S, O)
        dtw, dx = ops.butterfly_multiply_bw(tw, x, torch.empty(0, S, n, dtype=tdt, device="cuda"), True)
        assert dx.shape == (0, S, n) and dtw.shape == tw.shape and not dtw.any()
        y = ops.butterfly_multiply(tw, x, False, O)
        dtw, dx = torch.autograd.grad(y, (tw, x), g)
        assert y.shape == (0, S, O) and dx.shape == (0, S, n) and not dtw.any()
        bias = torch.randn(S, O, dtype=tdt, device="cuda", requires_grad=True)
        table = torch.randperm(n, device="cuda").int()
        y = ops.butterfly_multiply_perm(tw, x, table, None, bias, True, O)
        dtw, dx, db = torch.autograd.grad(y, (tw, x, bias), g)
        assert y.shape == (0, S, O) and dx.shape == (0, S, n) and not dtw.any() and not db.any()
        if L <= 12:
            tw4 = torch.randn(S, nb, L // 2, n // 4, 4, 4, dtype=tdt, device="cuda", requires_grad=True)
            tw2 = torch.randn(S, nb, L % 2, n // 2, 2, 2, dtype=tdt, device="cuda", requires_grad=True)
            y = ops.butterfly_multiply_base4(tw4, tw2, x, True, O)
            d4, d2, dx = torch.autograd.grad(y, (tw4, tw2, x), g, allow_unused=True)
            assert y.shape == (0, S, O) and dx.shape == (0, S, n) and not d4.any()
            assert d2 is None or not d2.any()
    torch.cuda.synchronize()


@pytest.mark.parametrize("L,nb", [(3, 1), (10, 2), (12, 2)])
def test_empty_rows(L, nb):
    """Rows of no input columns (everything is padding: the output is the bias or zero, d_input is
    empty, d_twiddle zero) and of no output columns (empty output; a zero gradient flows back)."""
    import butterfly_amd  # noqa: F401
    ops = torch.ops.torch_butterfly
    n = 1 << L
    B, S = 37, 2
    for tdt in (torch.float32, torch.complex64):
        say("empty rows", L, nb, tdt)
        tw = torch.randn(S, nb, L, n // 2, 2, 2, dtype=tdt, device="cuda", requires_grad=True)
        x0 = torch.empty(B, S, 0, dtype=tdt, device="cuda", requires_grad=True)
        g = torch.randn(B, S, n, dtype=tdt, device="cuda")
        y = ops.butterfly_multiply(tw, x0, True, None)
        dtw, dx = torch.autograd.grad(y, (tw, x0), g)
        assert y.shape == (B, S, n) and not y.any() and dx.shape == (B, S, 0) and not dtw.any()
        x = torch.randn(B, S, n, dtype=tdt, device="cuda", requires_grad=True)
        y = ops.butterfly_multiply(tw, x, False, 0)
        assert y.shape == (B, S, 0)
        dtw, dx = torch.autograd.grad(y, (tw, x), torch.empty(B, S, 0, dtype=tdt, device="cuda"))
        assert dx.shape == (B, S, n) and not dx.any() and not dtw.any()
    torch.cuda.synchronize()


def test_operator_errors():
    import butterfly_amd  # noqa: F401
    ops = torch.ops.torch_butterfly
    tw = torch.randn(1, 1, 3, 4, 2, 2, device="cuda")
    x = torch.randn(2, 1, 8, device="cuda")
    with pytest.raises(RuntimeError, match="must have shape"):
        ops.butterfly_multiply_fw(tw[:, :, :, :3], x, True, None)
    with pytest.raises(RuntimeError, match="output_size must be <= n"):
        ops.butterfly_multiply_fw(tw, x, True, 9)
    with pytest.raises(RuntimeError, match="same device"):
        ops.butterfly_multiply_fw(tw.cpu(), x, True, None)
    with pytest.raises(RuntimeError, match="float32 and complex64"):
        ops.butterfly_multiply_fw(tw.double(), x.double(), True, None)
    with pytest.raises(RuntimeError, match="must have dimension"):
        ops.butterfly_multiply_bw(tw, x, torch.randn(2, 8, device="cuda"), True)


def test_backward_is_bitwise_reproducible():
    """No atomics in the d_twiddle reduction: two runs give identical bits."""
    from butterfly_amd import _capi
    rng = np.random.default_rng(31)
    tw, x, g = make_case(rng, np.float32, 4096, 1, 10, 2)
    twd, xd, gd = dev(tw), dev(x), dev(g)
    say("determinism")
    a = _capi.multiply_bw(twd, xd, gd, False)
    b = _capi.multiply_bw(twd, xd, gd, False)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_headline_size_properties():
    """Batch 16384, n = 1024, nblocks = 2, decreasing stride first, through size-independent
    properties (the element-by-element comparison of all 16384 rows with the oracle is
    test_gpu_quoted_configs.py::test_headline_shape_at_full_size): (i) a 512-row slice against
    the oracle, (ii) the adjoint identity <y, g> = <x, d_input>, (iii) d_twiddle equals the sum
    of d_twiddle over batch chunks (rows are independent)."""
    from butterfly_amd import _capi
    rng = np.random.default_rng(41)
    B, L, nb = 16384, 10, 2
    tw, x, g = make_case(rng, np.float32, B, 1, L, nb)
    twd, xd, gd = dev(tw), dev(x), dev(g)
    say("headline fw")
    y = _capi.multiply_fw(twd, xd, False)
    say("headline bw")
    dtw, dx = _capi.multiply_bw(twd, xd, gd, False)
    torch.cuda.synchronize()
    sl = slice(7000, 7512)
    assert rel_err(y[sl].cpu().numpy(), oracle.butterfly_fw(tw, x[sl], False)) < FW_TOL
    _, dx_ref = oracle.butterfly_bw(tw, x[sl], g[sl], False)
    assert rel_err(dx[sl].cpu().numpy(), dx_ref) < BW_TOL
    lhs = torch.sum(y.double() * gd.double()).item()
    rhs = torch.sum(xd.double() * dx.double()).item()
    assert abs(lhs - rhs) < 1e-5 * abs(lhs) + 1e-2
    parts = [_capi.multiply_bw(twd, xd[i:i + 4096], gd[i:i + 4096], False)[0].double() for i in range(0, B, 4096)]
    assert rel_err(dtw.cpu().numpy(), sum(parts).cpu().numpy()) < BW_TOL
    dtw_ref, _ = oracle.butterfly_bw(tw, x[:1024], g[:1024], False)
    dtw_small, _ = _capi.multiply_bw(twd, xd[:1024], gd[:1024], False)
    assert rel_err(dtw_small.cpu().numpy(), dtw_ref) < BW_TOL


BIAS_CASES = [
    # dtype, B, S, L, nb, I, O, inc -- every kind of last pass: fast (fused), wide (fused),
    # span and generic (separate add), several stacks, trimmed outputs
    (np.float32, 37, 2, 5, 2, 20, 27, True),
    (np.float32, 300, 1, 10, 2, None, None, False),
    (np.float32, 41, 3, 7, 1, None, 100, True),
    (np.float32, 19, 1, 11, 2, None, 2000, False),
    (np.float32, 23, 2, 12, 1, None, None, True),
    (np.complex64, 29, 2, 6, 3, None, 50, False),
    (np.complex64, 17, 1, 11, 1, None, None, True),
    (np.complex64, 9, 1, 12, 1, None, 4000, True),
    (np.float32, 11, 1, 13, 1, None, 8000, True),
    (np.float32, 5000, 1, 10, 1, None, 1000, True),
    (np.float32, 2100, 1, 12, 2, None, 4090, True),
    (np.float32, 40, 1, 11, 1, None, 2000, True),        # whole-block forward kernel at any batch
    (np.complex64, 300, 1, 11, 1, None, None, False),
]


@pytest.mark.parametrize("case", BIAS_CASES, ids=lambda c: f"{np.dtype(c[0]).name}-B{c[1]}-S{c[2]}-L{c[3]}-nb{c[4]}-I{c[5]}-O{c[6]}-inc{int(c[7])}")
def test_bias_folded_into_forward_and_bias_gradient(case):
    """output = multiply + bias (one rounding of the sum, like the oracle's) and
    d_bias = column sums of grad, through the C ABI."""
    from butterfly_amd import _capi
    dtype, B, S, L, nb, I, O, inc = case
    say("bias case", case)
    rng = np.random.default_rng(1700 + L * 19 + nb)
    tw, x, g = make_case(rng, dtype, B, S, L, nb, I, O)
    cols = (1 << L) if O is None else O
    bias = randn(rng, (S, cols), dtype)
    y_ref = oracle.butterfly_fw(tw, x, inc, O) + bias[None]
    y = _capi.multiply_bias_fw(dev(tw), dev(x), dev(bias), inc, O)
    db = _capi.bias_grad(dev(g))
    torch.cuda.synchronize()
    assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL
    db_ref = g.astype(np.complex128 if np.iscomplexobj(g) else np.float64).sum(axis=0)
    assert rel_err(db.cpu().numpy(), db_ref) < BW_TOL
    # non-contiguous gradient, run-to-run bitwise equality
    gt = dev(np.ascontiguousarray(g.transpose(1, 0, 2))).transpose(0, 1)
    db2 = _capi.bias_grad(gt)
    db3 = _capi.bias_grad(gt)
    torch.cuda.synchronize()
    assert torch.equal(db2, db3) and torch.equal(db2, db)
    # the backward call that forms d_bias on the way
    dtw_ref, dx_ref = oracle.butterfly_bw(tw, x, g, inc)
    dtw, dx, db4 = _capi.multiply_bias_bw(dev(tw), dev(x), dev(g), inc)
    torch.cuda.synchronize()
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL
    assert rel_err(db4.cpu().numpy(), db_ref) < BW_TOL


def test_bias_operator_autograd():
    """The autograd operator returns the three gradients the separate formulation gives."""
    import butterfly_amd  # noqa: F401
    ops = torch.ops.torch_butterfly
    torch.manual_seed(5)
    for dtype, S, L, nb, O in [(torch.float32, 2, 6, 2, 50), (torch.complex64, 1, 5, 1, None),
                               (torch.float32, 1, 12, 2, None)]:
        n = 1 << L
        cols = n if O is None else O
        tw = (torch.randn(S, nb, L, n // 2, 2, 2, dtype=dtype) / 2 ** 0.5).cuda().requires_grad_()
        x = torch.randn(21, S, n, dtype=dtype).cuda().requires_grad_()
        bias = torch.randn(S, cols, dtype=dtype).cuda().requires_grad_()
        g = torch.randn(21, S, cols, dtype=dtype).cuda()
        y = ops.butterfly_multiply_bias(tw, x, bias, True, O)
        d_tw, d_x, d_b = torch.autograd.grad(y, (tw, x, bias), g)
        y2 = ops.butterfly_multiply(tw, x, True, O) + bias
        e_tw, e_x, e_b = torch.autograd.grad(y2, (tw, x, bias), g)
        for a, b in [(y, y2), (d_tw, e_tw), (d_x, e_x), (d_b, e_b)]:
            assert (a - b).abs().max().item() <= 1e-4 * max(1.0, b.abs().max().item())
    with pytest.raises(RuntimeError, match="bias must have shape"):
        ops.butterfly_multiply_bias_fw(tw.detach(), x.detach(), bias.detach()[:, :-1], True, None)


PERM_CASES = [
    # dtype, B, S, L, nb, I, O, inc, tables ("io" = both, "i", "o"), bias -- every kind of first
    # and last pass: register and LDS row fetch, wide, span, generic; padded inputs,
    # trimmed outputs, several stacks
    (np.float32, 37, 1, 5, 2, 20, 27, True, "io", True),
    (np.float32, 300, 1, 10, 2, None, None, False, "io", True),
    (np.float32, 41, 3, 7, 1, 100, None, True, "i", True),
    (np.float32, 2100, 1, 10, 1, None, 1000, True, "io", False),
    (np.complex64, 29, 1, 6, 3, None, 50, False, "io", True),
    (np.complex64, 530, 1, 10, 1, None, None, True, "io", False),
    (np.complex64, 130, 2, 9, 2, None, None, False, "i", False),
    (np.float32, 19, 1, 11, 2, None, 2000, False, "io", True),
    (np.float32, 23, 1, 12, 1, 4000, None, True, "io", False),
    (np.complex64, 17, 1, 11, 1, None, None, True, "io", True),
    (np.complex64, 9, 1, 12, 1, None, 4000, True, "o", False),
    (np.float32, 11, 1, 13, 1, None, 8000, True, "io", True),
    (np.float32, 7, 1, 14, 2, 16000, None, False, "io", False),
    (np.float32, 40, 1, 11, 1, None, 2000, True, "io", True),      # whole-block forward kernel
    (np.complex64, 300, 1, 11, 1, None, None, False, "io", False),
]


@pytest.mark.parametrize("case", PERM_CASES, ids=lambda c: f"{np.dtype(c[0]).name}-B{c[1]}-S{c[2]}-L{c[3]}-nb{c[4]}-I{c[5]}-O{c[6]}-inc{int(c[7])}-{c[8]}-bias{int(c[9])}")
def test_permutations_folded_into_first_read_and_last_write(case):
    """multiply_perm_fw / _bw through the C ABI against the oracle applied between explicit
    gathers: u = pad(x)[in_perm], y = B u + bias, out[out_index[c]] = y[c]."""
    from butterfly_amd import _capi
    dtype, B, S, L, nb, I, O, inc, which, with_bias = case
    say("perm case", case)
    n = 1 << L
    rng = np.random.default_rng(2300 + L * 23 + nb)
    tw, x, g = make_case(rng, dtype, B, S, L, nb, I, O)
    cols = n if O is None else O
    width = n if I is None else I
    # in front: a permutation of the `width` input columns, fixed points on the padding;
    # behind: a permutation of the `cols` output columns
    in_perm = np.arange(n)
    in_perm[:width] = rng.permutation(width)
    q = np.arange(n)
    q[:cols] = rng.permutation(cols)          # FixedPermutation(q): out[i] = y[q[i]]
    out_index = np.empty(n, dtype=np.int64)
    out_index[q] = np.arange(n)
    use_in, use_out = "i" in which, "o" in which
    bias = randn(rng, (S, cols), dtype) if with_bias else None

    xp = np.zeros((B, S, n), dtype=dtype)
    xp[:, :, :width] = x
    u = xp[:, :, in_perm] if use_in else xp
    y_ref = oracle.butterfly_fw(tw, u, inc, O)
    if with_bias:
        y_ref = y_ref + bias[None]
    out_ref = y_ref[:, :, q[:cols]] if use_out else y_ref
    gy = np.zeros((B, S, n), dtype=dtype)
    if use_out:
        gy[:, :, q[:cols]] = g               # y[q[i]] receives grad[i]
    else:
        gy[:, :, :cols] = g
    dtw_ref, du_ref = oracle.butterfly_bw(tw, u, gy[:, :, :cols], inc)
    dx_ref = np.zeros((B, S, n), dtype=du_ref.dtype)
    if use_in:
        dx_ref[:, :, in_perm] = du_ref
    else:
        dx_ref = du_ref
    dx_ref = dx_ref[:, :, :width]
    db_ref = gy[:, :, :cols].astype(np.complex128 if np.iscomplexobj(g) else np.float64).sum(axis=0)

    t_in = torch.from_numpy(in_perm.astype(np.int32)).cuda() if use_in else None
    t_out = torch.from_numpy(out_index.astype(np.int32)).cuda() if use_out else None
    xd, gd, twd = dev(x), dev(g), dev(tw)
    out = _capi.multiply_perm_fw(twd, xd, t_in, t_out, None if bias is None else dev(bias), inc, O)
    dtw, dx, db = _capi.multiply_perm_bw(twd, xd, gd, t_in, t_out, inc, with_bias)
    torch.cuda.synchronize()
    assert rel_err(out.cpu().numpy(), out_ref) < FW_TOL
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL
    if with_bias:
        assert rel_err(db.cpu().numpy(), db_ref) < BW_TOL
    # identity tables change nothing, bit for bit
    eye = torch.arange(n, dtype=torch.int32).cuda()
    plain = _capi.multiply_fw(twd, xd, inc, O)
    same = _capi.multiply_perm_fw(twd, xd, eye, eye, None, inc, O)
    torch.cuda.synchronize()
    assert torch.equal(plain, same)


def test_perm_operator_autograd_and_checks():
    """The autograd operator equals gather -> multiply -> + bias -> gather under autograd."""
    import butterfly_amd  # noqa: F401
    ops = torch.ops.torch_butterfly
    torch.manual_seed(9)
    for dtype, S, L, nb, O, with_bias in [(torch.float32, 1, 6, 2, 50, True), (torch.complex64, 1, 10, 1, None, False),
                                          (torch.float32, 1, 12, 2, None, True)]:
        n = 1 << L
        cols = n if O is None else O
        tw = (torch.randn(S, nb, L, n // 2, 2, 2, dtype=dtype) / 2 ** 0.5).cuda().requires_grad_()
        x = torch.randn(21, S, n, dtype=dtype).cuda().requires_grad_()
        bias = torch.randn(S, cols, dtype=dtype).cuda().requires_grad_() if with_bias else None
        g = torch.randn(21, S, cols, dtype=dtype).cuda()
        p_in = torch.randperm(n).cuda()
        q = torch.randperm(cols).cuda()
        full_q = torch.cat((q, torch.arange(cols, n).cuda()))
        out_index = torch.empty_like(full_q)
        out_index[full_q] = torch.arange(n).cuda()
        y = ops.butterfly_multiply_perm(tw, x, p_in.int(), out_index.int(), bias, True, O)
        wrt = (tw, x) + ((bias,) if with_bias else ())
        got = torch.autograd.grad(y, wrt, g)
        y2 = ops.butterfly_multiply(tw, x[..., p_in], True, O)
        if with_bias:
            y2 = y2 + bias
        y2 = y2[..., q]
        want = torch.autograd.grad(y2, wrt, g)
        for a, b in [(y, y2)] + list(zip(got, want)):
            assert (a - b).abs().max().item() <= 1e-4 * max(1.0, b.abs().max().item())
    with pytest.raises(RuntimeError, match="int32"):
        ops.butterfly_multiply_perm_fw(tw.detach(), x.detach(), p_in, None, None, True, None)
    with pytest.raises(RuntimeError, match="n entries"):
        ops.butterfly_multiply_perm_fw(tw.detach(), x.detach(), p_in.int()[:-1], None, None, True, None)


@pytest.mark.parametrize("shape", [(600, 1, 10, 2, False), (300, 1, 12, 2, True), (100, 2, 11, 1, False)],
                         ids=lambda s: f"B{s[0]}-S{s[1]}-L{s[2]}-nb{s[3]}")
def test_library_calls_replay_from_a_captured_graph(shape):
    """The library neither allocates nor synchronises, so its calls can be recorded in a HIP
    graph; every replay (with eager work and synchronisation in between) must reproduce what
    the eager calls give for the operands then in place."""
    from butterfly_amd import _capi
    B, S, L, nb, inc = shape
    n = 1 << L
    say("graph case", shape)
    torch.manual_seed(21)
    tw = (torch.randn(S, nb, L, n // 2, 2, 2) / 2 ** 0.5).cuda()
    x = torch.randn(B, S, n).cuda()
    g = torch.randn(B, S, n).cuda()
    bias = torch.randn(S, n).cuda()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):     # warm-up outside the capture, as graphs require
        _capi.multiply_bias_fw(tw, x, bias, inc)
        _capi.multiply_bias_bw(tw, x, g, inc)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = _capi.multiply_bias_fw(tw, x, bias, inc)
        dtw, dx, db = _capi.multiply_bias_bw(tw, x, g, inc)
    for rep in range(3):
        x.copy_(torch.randn(B, S, n).cuda())
        g.copy_(torch.randn(B, S, n).cuda())
        graph.replay()
        torch.cuda.synchronize()
        y_e = _capi.multiply_bias_fw(tw, x, bias, inc)
        dtw_e, dx_e, db_e = _capi.multiply_bias_bw(tw, x, g, inc)
        torch.cuda.synchronize()
        assert torch.equal(y, y_e) and torch.equal(dx, dx_e) and torch.equal(dtw, dtw_e) and torch.equal(db, db_e), rep


def test_scale_twiddle_through_the_c_abi():
    """Diagonals folded into the end factors: the library's result against a direct numpy
    evaluation of diag(out) (factor) diag(in) entry by entry, its gradients against the sums
    that definition gives (complex ones with the conjugates PyTorch's convention puts there),
    and the operator's autograd wiring."""
    from butterfly_amd import _capi
    import butterfly_amd  # noqa: F401
    rng = np.random.default_rng(21)

    def element(p, pos, stride):
        return (p // stride) * 2 * stride + pos * stride + p % stride

    cases = [(np.float32, True, 1, 1, 1, 2, 2), (np.float32, False, 2, 1, 1, 1, 3), (np.complex64, True, 2, 2, 3, 7, 15),
             (np.float32, False, 1, 2, 10, 1024, 1000), (np.complex64, False, 3, 3, 5, 32, 96), (np.float32, True, 2, 4, 4, 0, 32)]
    for dtype, inc, S, nb, L, in_len, out_len in cases:
        n = 1 << L
        for use_in, use_out in [(True, True), (True, False), (False, True)]:
            say("scale_twiddle", np.dtype(dtype).name, inc, S, nb, L, in_len, out_len, use_in, use_out)
            tw = randn(rng, (S, nb, L, n // 2, 2, 2), dtype)
            d = randn(rng, (in_len,), dtype) if use_in else None
            e = randn(rng, (out_len,), dtype) if use_out else None
            g = randn(rng, tw.shape, dtype)
            fin = np.ones((S, nb * L, n // 2, 2, 2), np.complex128)
            fout = np.ones_like(fin)
            s_first = 1 if inc else n // 2
            s_last = n // 2 if (inc != ((nb - 1) % 2 == 1)) else 1
            p = np.arange(n // 2)
            for pos in range(2):
                if d is not None:
                    idx = element(p, pos, s_first)
                    fin[:, 0, :, :, pos] = np.where(idx < in_len, np.concatenate([d, np.ones(n)])[idx], 1)[None, :, None]
                if e is not None:
                    for s in range(S):
                        idx = s * n + element(p, pos, s_last)
                        fout[s, -1, :, pos, :] = np.where(idx < out_len, np.concatenate([e, np.ones(S * n)])[idx], 1)[:, None]
            flat = tw.reshape(fin.shape).astype(np.complex128)
            ref = (flat * fin * fout).reshape(tw.shape)
            dev = lambda a: None if a is None else torch.from_numpy(a).cuda()
            got = _capi.scale_twiddle(dev(tw), dev(d), dev(e), inc).cpu().numpy()
            assert rel_err(got, ref) < 1e-6
            gf = g.reshape(fin.shape).astype(np.complex128)
            d_tw_ref = (gf * np.conj(fin * fout)).reshape(tw.shape)
            d_tw, d_in, d_out = _capi.scale_twiddle_bw(dev(tw), dev(d), dev(e), inc, dev(g))
            assert rel_err(d_tw.cpu().numpy(), d_tw_ref) < 1e-6
            if d is not None and in_len:
                contrib = gf[:, 0] * np.conj(flat[:, 0] * fout[:, 0])          # (S, n/2, r, c)
                d_in_ref = np.zeros(n, np.complex128)
                for pos in range(2):
                    np.add.at(d_in_ref, element(p, pos, s_first), contrib[:, :, :, pos].sum(axis=(0, 2)))
                assert rel_err(d_in.cpu().numpy(), d_in_ref[:in_len]) < 1e-5
            if e is not None and out_len:
                contrib = gf[:, -1] * np.conj(flat[:, -1] * fin[:, -1])
                d_out_ref = np.zeros((S, n), np.complex128)
                for pos in range(2):
                    d_out_ref[:, element(p, pos, s_last)] += contrib[:, :, pos, :].sum(axis=2)
                assert rel_err(d_out.cpu().numpy(), d_out_ref.reshape(-1)[:out_len]) < 1e-5
            # the operator under autograd returns the same three gradients
            t = dev(tw).requires_grad_()
            dd = None if d is None else dev(d).requires_grad_()
            ee = None if e is None else dev(e).requires_grad_()
            y = torch.ops.torch_butterfly.butterfly_scale_twiddle(t, dd, ee, inc)
            leaves = [v for v in (t, dd, ee) if v is not None]
            grads = torch.autograd.grad(y, leaves, dev(g))
            assert torch.equal(grads[0], d_tw)
            if dd is not None:
                assert torch.equal(grads[1], d_in)
            if ee is not None:
                assert torch.equal(grads[-1], d_out)
    with pytest.raises(RuntimeError):
        torch.ops.torch_butterfly.butterfly_scale_twiddle(torch.randn(1, 1, 3, 4, 2, 2).cuda(),
                                                          torch.randn(9).cuda(), None, True)


def test_misaligned_twiddle_is_rejected():
    """The kernels read the factor blocks with 16-byte loads; the library refuses a twiddle (or
    d_twiddle) that is not 16-byte aligned instead of launching on it."""
    from butterfly_amd import _capi
    L, nb, B = 6, 2, 5
    n = 1 << L
    shape = (1, nb, L, n // 2, 2, 2)
    numel = nb * L * (n // 2) * 4
    big = torch.randn(numel + 4, device="cuda")
    tw = big[1:1 + numel].view(shape)            # contiguous, 4 bytes off a 16-byte boundary
    assert tw.is_contiguous() and tw.data_ptr() % 16 == 4
    x = torch.randn(B, 1, n, device="cuda")
    with pytest.raises(_capi.ButterflyError, match="16-byte aligned"):
        _capi.multiply_fw(tw, x, True)
    with pytest.raises(_capi.ButterflyError, match="16-byte aligned"):
        _capi.multiply_bw(tw, x, torch.randn_like(x), True)
    # through the operator the shim's dense copy of a view is a fresh, aligned allocation
    import butterfly_amd  # noqa: F401
    y = torch.ops.torch_butterfly.butterfly_multiply_fw(tw, x, True, None)
    assert rel_err(y.cpu().numpy(), oracle.butterfly_fw(tw.cpu().numpy(), x.cpu().numpy(), True)) < FW_TOL
    # the aligned base-4 kernels read a thread's factor row with one 16-byte load
    numel4 = (L // 2) * (n // 4) * 16
    big4 = torch.randn(numel4 + 4, device="cuda")
    tw4 = big4[1:1 + numel4].view(1, 1, L // 2, n // 4, 4, 4)
    tw2 = torch.zeros(1, 1, 0, n // 2, 2, 2, device="cuda")
    assert tw4.is_contiguous() and tw4.data_ptr() % 16 == 4
    with pytest.raises(_capi.ButterflyError, match="16-byte aligned"):
        _capi.multiply_base4_fw(tw4, tw2, x, True)
    with pytest.raises(_capi.ButterflyError, match="16-byte aligned"):
        _capi.multiply_base4_bw(tw4, tw2, x, torch.randn_like(x), True)
    y4 = torch.ops.torch_butterfly.butterfly_multiply_base4_fw(tw4, tw2, x, True, None)
    assert rel_err(y4.cpu().numpy(), oracle.butterfly_base4_fw(tw4.cpu().numpy(), tw2.cpu().numpy(), x.cpu().numpy(), True)) < FW_TOL


SAVING_CASES = [
    # dtype, B, S, L, nb, I, O, inc -- backward plans of several passes: the forward keeps what they need
    (np.float32, 40, 2, 9, 3, None, None, True),
    (np.float32, 33, 1, 10, 5, 1000, 900, False),
    (np.float32, 21, 2, 11, 1, None, None, False),
    (np.float32, 21, 1, 11, 2, 2000, 1500, True),
    (np.float32, 300, 1, 12, 2, None, None, True),
    (np.float32, 1500, 1, 12, 1, None, None, False),
    (np.float32, 10, 2, 12, 3, 2 * 4096 + 7, 4091, False),
    (np.float32, 3, 1, 14, 1, None, None, True),
    (np.complex64, 40, 1, 9, 2, None, None, False),
    (np.complex64, 10, 2, 12, 3, None, None, True),
    (np.complex64, 600, 1, 12, 1, 4000, None, True),
    # the kernels the quoted 4096-wide configurations are timed through: two row groups in flight
    # (16 or more row groups per workgroup) on two blocks of 4096, both stride orders, and the
    # complex64 one-block plan at a batch that fills every workgroup
    (np.float32, 4200, 1, 12, 2, None, None, True),
    (np.float32, 4200, 1, 12, 2, None, None, False),
    (np.complex64, 2048, 1, 12, 1, None, None, True),
]


@pytest.mark.parametrize("case", SAVING_CASES, ids=lambda c: f"{np.dtype(c[0]).name}-B{c[1]}-S{c[2]}-L{c[3]}-nb{c[4]}-I{c[5]}-O{c[6]}-inc{int(c[7])}")
def test_forward_that_saves_for_the_backward(case):
    """bf_butterfly_multiply_fw_saving + bf_butterfly_multiply_bw_saved (the forward runs along the
    backward's pass plan and keeps the activations between the passes; the backward reads them
    instead of recomputing): all results against the oracle, with and without the bias."""
    from butterfly_amd import _capi
    dtype, B, S, L, nb, I, O, inc = case
    say("saving case", case)
    rng = np.random.default_rng(7000 + L * 17 + nb)
    tw, x, g = make_case(rng, dtype, B, S, L, nb, I, O)
    y_ref = oracle.butterfly_fw(tw, x, inc, O)
    dtw_ref, dx_ref = oracle.butterfly_bw(tw, x, g, inc)
    r = _capi.multiply_fw_bw_saving(dev(tw), dev(x), dev(g), inc, O)
    assert r is not None
    y, dtw, dx, _ = r
    torch.cuda.synchronize()
    assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL
    bias = randn(rng, (S, g.shape[2]), dtype)
    y, dtw, dx, db = _capi.multiply_fw_bw_saving(dev(tw), dev(x), dev(g), inc, O, bias=dev(bias))
    assert rel_err(y.cpu().numpy(), y_ref + bias[None]) < FW_TOL
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL
    assert rel_err(db.cpu().numpy(), g.sum(0)) < BW_TOL


def test_single_pass_problems_save_nothing():
    from butterfly_amd import _capi
    rng = np.random.default_rng(7100)
    tw, x, g = make_case(rng, np.float32, 50, 1, 10, 2)
    assert _capi.multiply_fw_bw_saving(dev(tw), dev(x), dev(g), False) is None


@pytest.mark.parametrize("dtype,L,nb", [(np.float32, 12, 2), (np.complex64, 12, 1), (np.float32, 10, 3)],
                         ids=["f32-4096-nb2", "c64-4096", "f32-1024-nb3"])
def test_autograd_operators_keep_activations_between_passes(dtype, L, nb):
    """torch.ops.torch_butterfly.butterfly_multiply / _bias under autograd (kept activations) against
    the oracle and against the operators called one by one (which recompute)."""
    import butterfly_amd  # noqa: F401
    ops = torch.ops.torch_butterfly
    rng = np.random.default_rng(7200 + L + nb)
    B, S, I, O = 70, 2, (1 << L) - 5, (1 << L) - 9
    tw, x, g = make_case(rng, dtype, B, S, L, nb, I, O)
    say("autograd keep", np.dtype(dtype).name, L, nb)
    y_ref = oracle.butterfly_fw(tw, x, True, O)
    dtw_ref, dx_ref = oracle.butterfly_bw(tw, x, g, True)
    twd, xd = dev(tw).requires_grad_(), dev(x).requires_grad_()
    y = ops.butterfly_multiply(twd, xd, True, O)
    assert y.shape == (B, S, O) and y.stride() == (S << L, 1 << L, 1)
    dtw, dx = torch.autograd.grad(y, (twd, xd), dev(g))
    assert rel_err(y.detach().cpu().numpy(), y_ref) < FW_TOL
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL
    dtw2, dx2 = ops.butterfly_multiply_bw(dev(tw), dev(x), dev(g), True)
    assert rel_err(dx.cpu().numpy(), dx2.cpu().numpy()) < 1e-6 and rel_err(dtw.cpu().numpy(), dtw2.cpu().numpy()) < 1e-6
    bias = randn(rng, (S, O), dtype)
    bd = dev(bias).requires_grad_()
    yb = ops.butterfly_multiply_bias(twd, xd, bd, True, O)
    dtw, dx, db = torch.autograd.grad(yb, (twd, xd, bd), dev(g))
    assert rel_err(yb.detach().cpu().numpy(), y_ref + bias[None]) < FW_TOL
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL
    assert rel_err(db.cpu().numpy(), g.sum(0)) < BW_TOL
    # no gradient wanted: nothing is kept, the plain forward plan runs
    with torch.no_grad():
        y0 = ops.butterfly_multiply(dev(tw), dev(x), True, O)
    assert rel_err(y0.cpu().numpy(), y_ref) < FW_TOL


@pytest.mark.parametrize("dtype,L,nb", [(np.complex64, 12, 1), (np.float32, 11, 2)], ids=["c64-4096", "f32-2048-nb2"])
def test_saving_forward_between_column_permutations(dtype, L, nb):
    """The pair that shares its activations with a permutation in front and behind (what
    special.fft(4096) under autograd runs): against the oracle between explicit gathers."""
    from butterfly_amd import _capi
    n = 1 << L
    rng = np.random.default_rng(7300 + L)
    B, S = 90, 1
    tw, x, g = make_case(rng, dtype, B, S, L, nb)
    in_perm = rng.permutation(n).astype(np.int32)
    out_index = rng.permutation(n).astype(np.int32)
    say("saving perm", np.dtype(dtype).name, L, nb)
    u = x[:, :, in_perm]
    y_mid = oracle.butterfly_fw(tw, u, False)
    y_ref = np.empty_like(y_mid)
    y_ref[:, :, out_index] = y_mid
    dtw_ref, du_ref = oracle.butterfly_bw(tw, u, g[:, :, out_index], False)
    dx_ref = np.zeros_like(x)
    dx_ref[:, :, in_perm] = du_ref
    y, dtw, dx, _ = _capi.multiply_fw_bw_saving(dev(tw), dev(x), dev(g), False, in_perm=dev(in_perm),
                                               out_index=dev(out_index))
    assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL


LONG_BASE4_CASES = [
    # dtype, B, S, L, nb, I, O, inc -- base-4 rows beyond one workgroup's registers: chunk + stage passes
    (np.float32, 37, 2, 11, 1, None, None, True),
    (np.float32, 37, 2, 11, 1, None, None, False),
    (np.float32, 300, 1, 12, 2, None, None, True),
    (np.float32, 300, 1, 12, 2, 4000, 4090, False),
    (np.float32, 21, 1, 13, 3, None, None, True),
    (np.float32, 21, 2, 13, 1, 2 * 8192 + 3, 8000, False),
    (np.float32, 9, 1, 14, 2, None, None, False),
    (np.float32, 2100, 1, 12, 1, None, None, True),
    (np.complex64, 41, 2, 9, 2, None, None, True),
    (np.complex64, 41, 1, 9, 3, 500, 490, False),
    (np.complex64, 600, 1, 10, 2, None, None, False),
    (np.complex64, 13, 2, 11, 1, None, None, True),
    (np.complex64, 13, 1, 12, 2, None, None, False),
    (np.float32, 5, 1, 16, 1, None, None, True),
    (np.float32, 2, 1, 19, 1, None, None, True),
    (np.complex64, 3, 1, 15, 1, None, None, False),
]


@pytest.mark.parametrize("case", LONG_BASE4_CASES, ids=lambda c: f"{np.dtype(c[0]).name}-B{c[1]}-S{c[2]}-L{c[3]}-nb{c[4]}-I{c[5]}-O{c[6]}-inc{int(c[7])}")
def test_base4_long_rows(case):
    from butterfly_amd import _capi
    dtype, B, S, L, nb, I, O, inc = case
    say("long base4 case", case)
    rng = np.random.default_rng(8000 + L * 7 + nb)
    n = 1 << L
    I_ = n if I is None else I
    tw4 = (randn(rng, (S, nb, L // 2, n // 4, 4, 4), dtype) / 2).astype(dtype)
    tw2 = (randn(rng, (S, nb, L % 2, n // 2, 2, 2), dtype) / np.sqrt(2)).astype(dtype)
    x = randn(rng, (B, S, I_), dtype)
    g = randn(rng, (B, S, n if O is None else O), dtype)
    y_ref = oracle.butterfly_base4_fw(tw4, tw2, x, inc, O)
    d4_ref, d2_ref, dx_ref = oracle.butterfly_base4_bw(tw4, tw2, x, g, inc)
    y = _capi.multiply_base4_fw(dev(tw4), dev(tw2), dev(x), inc, O)
    d4, d2, dx = _capi.multiply_base4_bw(dev(tw4), dev(tw2), dev(x), dev(g), inc)
    torch.cuda.synchronize()
    assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(d4.cpu().numpy(), d4_ref) < BW_TOL
    if L % 2:
        assert rel_err(d2.cpu().numpy(), d2_ref) < BW_TOL


SAVING4_CASES = [
    # dtype, B, S, L, nb, I, O, inc -- base-4 backward plans of several passes
    (np.float32, 700, 2, 8, 2, None, None, True),
    (np.float32, 90, 1, 10, 3, 1000, 900, False),
    (np.float32, 50, 2, 7, 2, None, None, False),
    (np.complex64, 60, 1, 6, 3, None, 50, True),
    (np.float32, 37, 1, 12, 1, None, None, True),
    (np.float32, 21, 2, 11, 2, 2000, 1500, False),
    (np.complex64, 13, 1, 10, 2, None, None, False),
]


@pytest.mark.parametrize("case", SAVING4_CASES, ids=lambda c: f"{np.dtype(c[0]).name}-B{c[1]}-S{c[2]}-L{c[3]}-nb{c[4]}-I{c[5]}-O{c[6]}-inc{int(c[7])}")
def test_base4_forward_that_keeps_activations(case):
    """The base-4 saving pair against the oracle and, bit for bit, against the plain calls (same
    kernels, the backward only skips its replay launches); the autograd operator uses it."""
    from butterfly_amd import _capi
    import butterfly_amd  # noqa: F401
    dtype, B, S, L, nb, I, O, inc = case
    say("base-4 saving case", case)
    rng = np.random.default_rng(8100 + L * 7 + nb)
    n = 1 << L
    tw4 = (randn(rng, (S, nb, L // 2, n // 4, 4, 4), dtype) / 2).astype(dtype)
    tw2 = (randn(rng, (S, nb, L % 2, n // 2, 2, 2), dtype) / np.sqrt(2)).astype(dtype)
    x = randn(rng, (B, S, n if I is None else I), dtype)
    g = randn(rng, (B, S, n if O is None else O), dtype)
    t4, t2, xd, gd = dev(tw4), dev(tw2), dev(x), dev(g)
    res = _capi.multiply_base4_fw_bw_saving(t4, t2, xd, gd, inc, O)
    assert res is not None, "a plan of several passes keeps activations"
    y, d4, d2, dx = res
    y_p = _capi.multiply_base4_fw(t4, t2, xd, inc, O)
    d4_p, d2_p, dx_p = _capi.multiply_base4_bw(t4, t2, xd, gd, inc)
    torch.cuda.synchronize()
    assert torch.equal(y, y_p) and torch.equal(dx, dx_p) and torch.equal(d4, d4_p) and torch.equal(d2, d2_p)
    y_ref = oracle.butterfly_base4_fw(tw4, tw2, x, inc, O)
    d4_ref, d2_ref, dx_ref = oracle.butterfly_base4_bw(tw4, tw2, x, g, inc)
    assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(d4.cpu().numpy(), d4_ref) < BW_TOL
    if L % 2:
        assert rel_err(d2.cpu().numpy(), d2_ref) < BW_TOL
    # the operator under autograd gives the same bits
    a4, a2, ax = t4.clone().requires_grad_(), t2.clone().requires_grad_(), xd.clone().requires_grad_()
    ya = torch.ops.torch_butterfly.butterfly_multiply_base4(a4, a2, ax, inc, O)
    wrt = (a4, ax) + ((a2,) if L % 2 else ())
    grads = torch.autograd.grad(ya, wrt, gd)
    assert torch.equal(ya.detach(), y) and torch.equal(grads[0], d4) and torch.equal(grads[1], dx)
    if L % 2:
        assert torch.equal(grads[2], d2)


def test_base4_single_pass_saves_nothing():
    from butterfly_amd import _capi
    t4 = torch.randn(1, 1, 4, 64, 4, 4).cuda()
    t2 = torch.zeros(1, 1, 0, 128, 2, 2).cuda()
    x = torch.randn(10, 1, 256).cuda()
    assert _capi.multiply_base4_fw_bw_saving(t4, t2, x, torch.randn_like(x), True) is None


def test_two_streams_with_their_own_workspaces():
    """Two problems enqueued alternately on two streams (default priority), each call with a
    workspace of its own: the library keeps no state between calls, so both streams' results must
    equal the oracle's whatever the interleaving on the device."""
    from butterfly_amd import _capi
    rng = np.random.default_rng(7300)
    cases = [make_case(rng, np.float32, 3000, 1, 10, 2), make_case(rng, np.complex64, 300, 1, 12, 1)]
    incs = [False, True]
    refs = [(oracle.butterfly_fw(tw, x, inc), *oracle.butterfly_bw(tw, x, g, inc)) for (tw, x, g), inc in zip(cases, incs)]
    ops = [tuple(dev(a) for a in c) for c in cases]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    results = [[], []]
    say("two streams: enqueue")
    for rep in range(4):
        for k in (0, 1):
            with torch.cuda.stream(streams[k]):
                tw, x, g = ops[k]
                y = _capi.multiply_fw(tw, x, incs[k])
                dtw, dx = _capi.multiply_bw(tw, x, g, incs[k])
                results[k].append((y, dtw, dx))
    for s in streams:
        s.synchronize()
    torch.cuda.synchronize()
    say("two streams: check")
    for k in (0, 1):
        y_ref, dtw_ref, dx_ref = refs[k]
        for y, dtw, dx in results[k]:
            assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL
            assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
            assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL


def test_backward_checks_the_size_of_the_saved_area():
    """bf_butterfly_multiply_bw_saved is told how large the area behind `saved` is and refuses one
    that is smaller than the planes its own plan reads."""
    from butterfly_amd import _capi
    rng = np.random.default_rng(7400)
    tw, x, g = make_case(rng, np.float32, 20, 1, 12, 2)
    with pytest.raises(_capi.ButterflyError) as info:
        _capi.multiply_fw_bw_saving(dev(tw), dev(x), dev(g), True, saved_given=4096)
    assert info.value.code == _capi.BF_ERR_WORKSPACE
    torch.cuda.synchronize()


def test_autograd_backward_with_a_gradient_whose_plan_keeps_nothing():
    """The forward keeps activations for the backward plan it expects; a gradient that arrives as a
    view with a huge batch stride makes the backward plan differently (rows out of reach of 32-bit
    offsets -> the fallback kernels, which read no kept activations).  The operator then recomputes
    instead of failing."""
    import butterfly_amd  # noqa: F401
    ops = torch.ops.torch_butterfly
    rng = np.random.default_rng(7401)
    B, L, nb = 6, 11, 1
    n = 1 << L
    tw, x, g = make_case(rng, np.float32, B, 1, L, nb)
    twd, xd = dev(tw).requires_grad_(), dev(x).requires_grad_()
    y = ops.butterfly_multiply(twd, xd, True, None)
    # rows of the gradient 2^27 elements (512 MiB) apart: a view into a 3 GiB buffer
    stride = 1 << 27
    big = torch.empty(B * stride, dtype=torch.float32, device="cuda")
    gview = torch.as_strided(big, (B, 1, n), (stride, n, 1))
    gview.copy_(dev(g))
    say("autograd with strided gradient", gview.stride())
    # the premise: with these strides the backward keeps nothing, with dense ones it does
    from butterfly_amd import _capi
    p = _capi.make_problem(xd.detach(), L, nb, True, n)
    p.output_stride = _capi._strides(gview)
    p.d_input_stride = _capi._strides(xd.detach())
    assert _capi.lib().bf_butterfly_multiply_saved_bytes(ctypes.byref(p)) == 0
    p.output_stride = _capi._strides(dev(g))
    assert _capi.lib().bf_butterfly_multiply_saved_bytes(ctypes.byref(p)) > 0
    dtw, dx = torch.autograd.grad(y, (twd, xd), gview)
    torch.cuda.synchronize()
    dtw_ref, dx_ref = oracle.butterfly_bw(tw, x, g, True)
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL


@pytest.mark.parametrize("B", [1, 7, 64, 300, 1100])
def test_small_batches_of_the_inference_shapes(B):
    """The batch sizes of the reference's inference benchmarks (/root/reference/butterfly/benchmark_linear.py,
    torch_butterfly/input_padding_benchmark.py): 1024-wide rows with one and two blocks and the
    4096-wide two-block Linear drop-in, complex 1024.  At these sizes the backward call runs on
    fewer workgroups than compute units (fewer partial slices to write and reduce), so the row
    loops of its workgroups get longer than the batch alone would make them."""
    from butterfly_amd import _capi
    rng = np.random.default_rng(7500 + B)
    for dtype, L, nb, inc in [(np.float32, 10, 1, True), (np.float32, 10, 2, False), (np.float32, 12, 2, True),
                              (np.complex64, 10, 1, True), (np.float32, 7, 2, True)]:
        say("small batch", B, np.dtype(dtype).name, L, nb, inc)
        tw, x, g = make_case(rng, dtype, B, 1, L, nb)
        y_ref = oracle.butterfly_fw(tw, x, inc)
        dtw_ref, dx_ref = oracle.butterfly_bw(tw, x, g, inc)
        y = _capi.multiply_fw(dev(tw), dev(x), inc)
        dtw, dx = _capi.multiply_bw(dev(tw), dev(x), dev(g), inc)
        torch.cuda.synchronize()
        assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL
        assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
        assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL


@pytest.mark.parametrize("B,S,L,inc,I,O", [(16384, 1, 10, True, None, None), (13001, 1, 10, False, 1000, 700),
                                           (50000, 2, 8, False, None, None), (100003, 1, 7, True, None, None),
                                           (30000, 1, 9, True, None, None), (30000, 1, 9, False, None, None),
                                           (400000, 1, 4, False, None, None)],
                         ids=lambda v: str(v))
def test_forward_with_two_workgroups_per_compute_unit(B, S, L, inc, I, O):
    """Float passes over two blocks put two forward workgroups on every compute unit once each of
    them has enough rows (the 64-register variant of the kernel, two row sets in LDS): batches
    beyond that threshold for several row lengths, both stride orders, a ragged last group, padded
    and trimmed widths; forward and backward against the oracle.  (512-element rows with decreasing
    stride first stay on one workgroup per unit; they are here for the same sizes.)"""
    from butterfly_amd import _capi
    rng = np.random.default_rng(7100 + L + int(inc))
    tw, x, g = make_case(rng, np.float32, B, S, L, 2, I, O)
    say("paired forward case", B, S, L, inc, I, O)
    y_ref = oracle.butterfly_fw(tw, x, inc, O)
    twd, xd = dev(tw), dev(x)
    for rep in range(3):   # repeated calls: the row pipeline must not depend on timing
        y = _capi.multiply_fw(twd, xd, inc, O)
        torch.cuda.synchronize()
        assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL, (B, S, L, inc, rep)
    if B > 17000:      # (the scalar oracle's backward takes seconds per case at these sizes)
        return
    dtw_ref, dx_ref = oracle.butterfly_bw(tw, x, g, inc)
    dtw, dx = _capi.multiply_bw(twd, xd, dev(g), inc)
    torch.cuda.synchronize()
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL
    assert rel_err(dtw.cpu().numpy(), dtw_ref) < BW_TOL


@pytest.mark.parametrize("B,S,L,nb,inc,I,O", [(16384, 1, 10, 1, True, None, None), (70001, 1, 8, 2, False, 250, 200),
                                              (13000, 1, 10, 2, False, None, None), (40000, 3, 8, 1, True, None, None)],
                         ids=lambda v: str(v))
def test_base4_forward_with_two_workgroups_per_compute_unit(B, S, L, nb, inc, I, O):
    """The aligned base-4 forward kernels run two workgroups per compute unit for rows of 256 and
    1024 once each workgroup has enough rows: batches beyond that threshold, both stride orders,
    a ragged last group, padded and trimmed widths, against the oracle; calls repeated."""
    from butterfly_amd import _capi
    n = 1 << L
    I = n if I is None else I
    O = n if O is None else O
    rng = np.random.default_rng(7300 + L + nb)
    say("paired base-4 forward case", B, S, L, nb, inc, I, O)
    tw4 = (randn(rng, (S, nb, L // 2, n // 4, 4, 4), np.float32) / 2).astype(np.float32)
    tw2 = np.zeros((S, nb, 0, n // 2, 2, 2), np.float32)
    x = randn(rng, (B, S, I), np.float32)
    y_ref = oracle.butterfly_base4_fw(tw4, tw2, x, inc, O)
    t4, t2, xd = dev(tw4), dev(tw2), dev(x)
    for rep in range(3):
        y = _capi.multiply_base4_fw(t4, t2, xd, inc, O)
        torch.cuda.synchronize()
        assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL, (B, S, L, nb, inc, rep)
