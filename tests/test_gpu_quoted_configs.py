"""Parity at the shapes the measurements are quoted on, at full size, and with many row groups
per workgroup: every figure of the benchmark then rests on results that were compared with the
CPU oracle element by element.  Through the C ABI; tolerances as elsewhere (max|err| / max|ref|:
1e-5 forward, 1e-4 gradients)."""
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


def check_base2(tw, x, g, inc, O=None, what=""):
    from butterfly_amd import _capi
    say("base-2 case", what, tw.dtype, x.shape, tw.shape[1], inc)
    twd, xd, gd = dev(tw), dev(x), dev(g)
    y = _capi.multiply_fw(twd, xd, inc, O)
    dtw, dx = _capi.multiply_bw(twd, xd, gd, inc)
    torch.cuda.synchronize()
    y, dtw, dx = y.cpu().numpy(), dtw.cpu().numpy(), dx.cpu().numpy()
    y_ref = oracle.butterfly_fw(tw, x, inc, O)
    assert rel_err(y, y_ref) < FW_TOL, what
    del y_ref
    dtw_ref, dx_ref = oracle.butterfly_bw(tw, x, g, inc)
    assert rel_err(dx, dx_ref) < BW_TOL, what
    assert rel_err(dtw, dtw_ref) < BW_TOL, what


def base2_operands(rng, dtype, B, S, L, nb):
    n = 1 << L
    tw = (randn(rng, (S, nb, L, n // 2, 2, 2), dtype) / np.sqrt(2)).astype(dtype)
    return tw, randn(rng, (B, S, n), dtype), randn(rng, (B, S, n), dtype)


def test_headline_shape_at_full_size():
    """(16384, 1, 1024) fp32, two blocks, decreasing stride first: output, d_input and d_twiddle
    of all 16384 rows against the oracle."""
    rng = np.random.default_rng(4101)
    tw, x, g = base2_operands(rng, np.float32, 16384, 1, 10, 2)
    check_base2(tw, x, g, False, what="headline")


def test_forward_only_shape_at_full_size():
    """(2048, 1, 1024) fp32, one block, increasing stride."""
    rng = np.random.default_rng(4102)
    tw, x, g = base2_operands(rng, np.float32, 2048, 1, 10, 1)
    check_base2(tw, x, g, True, what="forward-only shape")


@pytest.mark.parametrize("inc", [True, False], ids=["inc", "dec"])
def test_two_blocks_of_4096_with_two_row_groups_in_flight(inc):
    """(4200, 1, 4096) fp32, two blocks: with this many rows the backward passes on the high bits
    (two blocks meeting in bits 10, 11: one up-and-down span) and on the chunks run the variant
    that keeps two row groups in flight."""
    rng = np.random.default_rng(4103 + int(inc))
    tw, x, g = base2_operands(rng, np.float32, 4200, 1, 12, 2)
    check_base2(tw, x, g, inc, what="two blocks of 4096")


def test_dft_factors_at_4096_all_gradients():
    """complex64 n = 4096 with the factors of the normalised DFT: the output against numpy's FFT
    of the bit-reversed rows, and all three results (d_twiddle included) against the oracle."""
    from butterfly_amd import special
    from butterfly_amd.permutation import bitreversal_permutation
    L, B = 12, 2048
    n = 1 << L
    rng = np.random.default_rng(4105)
    tw = special.fft(n, normalized=True, with_br_perm=False).twiddle.detach().cpu().numpy()
    assert tw.dtype == np.complex64 and tw.shape == (1, 1, L, n // 2, 2, 2)
    x, g = randn(rng, (B, 1, n), np.complex64), randn(rng, (B, 1, n), np.complex64)
    check_base2(tw, x, g, True, what="DFT factors")
    from butterfly_amd import _capi
    br = np.asarray(bitreversal_permutation(n))
    y = _capi.multiply_fw(dev(tw), dev(x[:, :, br]), True, None).cpu().numpy()
    ref = np.fft.fft(x.astype(np.complex128), axis=-1, norm="ortho")
    assert rel_err(y, ref.astype(np.complex64)) < FW_TOL


def check_saving_pair(tw, x, g, inc, what=""):
    """The activation-keeping forward / backward pair (what the operator runs under autograd)
    against the oracle."""
    from butterfly_amd import _capi
    say("saving pair", what, tw.dtype, x.shape, tw.shape[1], inc)
    r = _capi.multiply_fw_bw_saving(dev(tw), dev(x), dev(g), inc, None)
    assert r is not None, "this problem keeps activations between its backward passes"
    y, dtw, dx, _ = r
    torch.cuda.synchronize()
    y, dtw, dx = y.cpu().numpy(), dtw.cpu().numpy(), dx.cpu().numpy()
    y_ref = oracle.butterfly_fw(tw, x, inc, None)
    assert rel_err(y, y_ref) < FW_TOL, what
    del y_ref
    dtw_ref, dx_ref = oracle.butterfly_bw(tw, x, g, inc)
    assert rel_err(dx, dx_ref) < BW_TOL, what
    assert rel_err(dtw, dtw_ref) < BW_TOL, what


def test_dft_factors_at_4096_through_the_activation_keeping_pair():
    """The complex64 FFT configuration the way its benchmark line is timed: forward that keeps the
    activation between the two backward passes, backward that starts from it; DFT factors, 2048
    rows (every workgroup of both passes walks several row groups)."""
    from butterfly_amd import special
    L, B = 12, 2048
    n = 1 << L
    rng = np.random.default_rng(4106)
    tw = special.fft(n, normalized=True, with_br_perm=False).twiddle.detach().cpu().numpy()
    x, g = randn(rng, (B, 1, n), np.complex64), randn(rng, (B, 1, n), np.complex64)
    check_saving_pair(tw, x, g, True, what="DFT factors, kept activations")


def test_fft_configuration_at_full_size():
    """(8192, 1, 4096) complex64 with the DFT factors, all 8192 rows: plain calls and the
    activation-keeping pair, output / d_input / d_twiddle against the oracle (whose backward
    scratch is 3 GiB here)."""
    from butterfly_amd import special
    L, B = 12, 8192
    n = 1 << L
    rng = np.random.default_rng(4107)
    tw = special.fft(n, normalized=True, with_br_perm=False).twiddle.detach().cpu().numpy()
    x, g = randn(rng, (B, 1, n), np.complex64), randn(rng, (B, 1, n), np.complex64)
    from butterfly_amd import _capi
    say("FFT configuration at full size")
    twd, xd, gd = dev(tw), dev(x), dev(g)
    y = _capi.multiply_fw(twd, xd, True, None).cpu().numpy()
    dtw, dx = (t.cpu().numpy() for t in _capi.multiply_bw(twd, xd, gd, True))
    ys, dtws, dxs, _ = _capi.multiply_fw_bw_saving(twd, xd, gd, True, None)
    torch.cuda.synchronize()
    ys, dtws, dxs = ys.cpu().numpy(), dtws.cpu().numpy(), dxs.cpu().numpy()
    del twd, xd, gd
    torch.cuda.empty_cache()
    y_ref = oracle.butterfly_fw(tw, x, True, None)
    assert rel_err(y, y_ref) < FW_TOL and rel_err(ys, y_ref) < FW_TOL
    del y_ref, y, ys
    dtw_ref, dx_ref = oracle.butterfly_bw(tw, x, g, True)
    assert rel_err(dx, dx_ref) < BW_TOL and rel_err(dxs, dx_ref) < BW_TOL
    assert rel_err(dtw, dtw_ref) < BW_TOL and rel_err(dtws, dtw_ref) < BW_TOL


@pytest.mark.parametrize("dtype", [np.float32, np.complex64], ids=["f32", "c64"])
@pytest.mark.parametrize("inc", [True, False], ids=["inc", "dec"])
def test_reference_race_condition_shape(dtype, inc):
    """The shape the reference's own test uses to provoke races in its d_twiddle reduction
    (/root/reference/tests/test_multiply.py:20-59): batch 8192, n = 512, 2 stacks, 3 blocks."""
    rng = np.random.default_rng(4110 + int(inc) + 2 * (np.dtype(dtype).kind == "c"))
    tw, x, g = base2_operands(rng, dtype, 8192, 2, 9, 3)
    check_base2(tw, x, g, inc, what="race-condition shape")


def check_base4(tw4, tw2, x, g, inc, O=None, what=""):
    from butterfly_amd import _capi
    say("base-4 case", what, x.shape, tw4.shape[1], inc)
    y = _capi.multiply_base4_fw(dev(tw4), dev(tw2), dev(x), inc, O)
    d4, d2, dx = _capi.multiply_base4_bw(dev(tw4), dev(tw2), dev(x), dev(g), inc)
    torch.cuda.synchronize()
    y_ref = oracle.butterfly_base4_fw(tw4, tw2, x, inc, O)
    d4_ref, d2_ref, dx_ref = oracle.butterfly_base4_bw(tw4, tw2, x, g, inc)
    assert rel_err(y.cpu().numpy(), y_ref) < FW_TOL, what
    assert rel_err(dx.cpu().numpy(), dx_ref) < BW_TOL, what
    assert rel_err(d4.cpu().numpy(), d4_ref) < BW_TOL, what
    if tw2.size:
        assert rel_err(d2.cpu().numpy(), d2_ref) < BW_TOL, what


def base4_operands(rng, B, S, L, nb, I=None, O=None):
    n = 1 << L
    tw4 = (randn(rng, (S, nb, L // 2, n // 4, 4, 4), np.float32) / 2).astype(np.float32)
    tw2 = np.zeros((S, nb, 0, n // 2, 2, 2), np.float32)
    return tw4, tw2, randn(rng, (B, S, n if I is None else I), np.float32), randn(rng, (B, S, n if O is None else O), np.float32)


@pytest.mark.parametrize("L", [2, 4, 6, 8, 10])
def test_base4_aligned_kernels_many_row_groups_per_workgroup(L):
    """Float, even log_n: enough rows that every workgroup of the aligned base-4 kernels goes
    round its row loop many times (prefetch one group ahead, alternating LDS buffers), with a
    ragged last group, both stride orders, one and two blocks."""
    n = 1 << L
    rng = np.random.default_rng(4200 + L)
    B = min(5000 * (1024 // n), 200000) + 3
    for nb in (1, 2):
        for inc in (True, False):
            tw4, tw2, x, g = base4_operands(rng, B, 1, L, nb)
            check_base4(tw4, tw2, x, g, inc, what=f"L={L} nb={nb} inc={inc} B={B}")
    # several stacks, padded input, trimmed output
    tw4, tw2, x, g = base4_operands(rng, 3001 * max(1, 256 // n), 3, L, 1, I=n + 3, O=max(1, n - 1))
    check_base4(tw4, tw2, x, g, True, O=max(1, n - 1), what=f"L={L} three stacks")


def test_base4_shape_at_full_size():
    """(16384, 4, 256) fp32 base-4, one block, increasing stride."""
    rng = np.random.default_rng(4300)
    tw4, tw2, x, g = base4_operands(rng, 16384, 4, 8, 1)
    check_base4(tw4, tw2, x, g, True, what="base-4 shape at full size")


@pytest.mark.parametrize("shape", [(200003, 1, 5, 1), (300001, 1, 4, 2), (120007, 2, 6, 1), (70001, 1, 6, 3)],
                         ids=lambda s: f"B{s[0]}-S{s[1]}-L{s[2]}-nb{s[3]}")
@pytest.mark.parametrize("inc", [True, False], ids=["inc", "dec"])
def test_complex_short_rows_many_row_groups_per_workgroup(shape, inc):
    """complex64 rows of 16 to 64 elements (what the low passes of longer complex rows and the
    small butterflies of KOP2d run on) and enough of them that every workgroup walks its row
    loop many times, with a ragged last group."""
    B, S, L, nb = shape
    rng = np.random.default_rng(4400 + L * 10 + nb + int(inc))
    tw, x, g = base2_operands(rng, np.complex64, B, S, L, nb)
    check_base2(tw, x, g, inc, what="complex short rows")
