"""CPU-only checks: the C ABI library loads and exports what the header declares, argument
validation, host-side twiddle algebra and module bookkeeping.  No kernel is launched."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from conftest import ROOT, randn, rel_err
from oracle import oracle


def header_functions():
    text = open(os.path.join(ROOT, "include", "butterfly_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bf_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from butterfly_amd import _capi
    names = header_functions()
    assert len(names) >= 11
    assert sorted(_capi.SYMBOLS) == names
    L = _capi.lib()
    for name in names:
        assert hasattr(L, name), name
    assert L.bf_version() >= 100
    assert L.bf_hip_version() > 0


def test_c_abi_rejects_bad_problems_on_the_host():
    from butterfly_amd import _capi
    L = _capi.lib()
    p = _capi.Problem()
    p.dtype, p.batch, p.nstacks, p.log_n, p.nblocks = 7, 1, 1, 3, 1
    p.input_size = p.output_size = 8
    null = ctypes.c_void_p(0)
    assert L.bf_butterfly_multiply_fw(ctypes.byref(p), null, null, null, null, 0, null) == -1
    assert b"dtype" in L.bf_last_error()
    p.dtype, p.output_size = 0, 9
    assert L.bf_butterfly_multiply_fw(ctypes.byref(p), null, null, null, null, 0, null) == -1
    assert b"output_size" in L.bf_last_error()
    p.output_size, p.log_n = 8, 31
    assert L.bf_butterfly_multiply_fw(ctypes.byref(p), null, null, null, null, 0, null) == -1
    p.log_n = 3
    p.input_stride[2] = -1
    assert L.bf_butterfly_multiply_bw(ctypes.byref(p), null, null, null, null, null, null, 0, null) == -1
    assert L.bf_butterfly_multiply_fw(None, null, null, null, null, 0, null) == -1
    # workspace query is pure host arithmetic
    p.input_stride[2] = 1
    p.batch, p.log_n, p.nblocks = 16384, 10, 2
    assert 0 < L.bf_butterfly_multiply_bw_workspace_bytes(ctypes.byref(p)) < _capi.SIZE_INVALID
    # ... and tells "no workspace needed" (0) from "not a valid problem" (BF_SIZE_INVALID)
    p.input_size = p.output_size = 1024
    for name in ("d_input_stride", "output_stride", "input_stride"):
        getattr(p, name)[0], getattr(p, name)[1], getattr(p, name)[2] = 1024, 1024, 1
    assert L.bf_butterfly_multiply_fw_workspace_bytes(ctypes.byref(p)) == 0
    assert L.bf_butterfly_multiply_saved_bytes(ctypes.byref(p)) == 0
    p.output_size = 1025
    queries = [L.bf_butterfly_multiply_fw_workspace_bytes, L.bf_butterfly_multiply_bw_workspace_bytes,
               L.bf_butterfly_multiply_saved_bytes, L.bf_butterfly_multiply_base4_fw_workspace_bytes,
               L.bf_butterfly_multiply_base4_bw_workspace_bytes, L.bf_butterfly_multiply_base4_saved_bytes,
               L.bf_butterfly_multiply_bias_bw_workspace_bytes, L.bf_butterfly_bias_grad_workspace_bytes,
               L.bf_butterfly_multiply_base4_bw_saved_workspace_bytes]
    for q in queries:
        assert q(ctypes.byref(p)) == _capi.SIZE_INVALID, q.__name__
        assert b"output_size" in L.bf_last_error()
    assert L.bf_butterfly_multiply_bw_saved_workspace_bytes(ctypes.byref(p), 0) == _capi.SIZE_INVALID
    with pytest.raises(_capi.ButterflyError):
        _capi._size(L.bf_butterfly_multiply_fw_workspace_bytes(ctypes.byref(p)))


def test_operator_schemas_and_host_side_checks():
    import butterfly_amd  # noqa: F401
    ops = torch.ops.torch_butterfly
    assert str(ops.butterfly_multiply_fw.default._schema) == \
        "torch_butterfly::butterfly_multiply_fw(Tensor _0, Tensor _1, bool _2, int? _3) -> Tensor _0"
    assert str(ops.butterfly_multiply_bw.default._schema) == \
        "torch_butterfly::butterfly_multiply_bw(Tensor _0, Tensor _1, Tensor _2, bool _3) -> (Tensor _0, Tensor _1)"
    assert str(ops.butterfly_multiply.default._schema) == \
        "torch_butterfly::butterfly_multiply(Tensor _0, Tensor _1, bool _2, int? _3) -> Tensor _0"
    assert ops.cuda_version() == -1 and ops.hip_version() > 0
    tw, x = torch.randn(1, 1, 3, 4, 2, 2), torch.randn(2, 1, 8)
    with pytest.raises(RuntimeError, match="must have shape"):
        ops.butterfly_multiply_fw(tw[:, :, :2], x, True, None)
    with pytest.raises(RuntimeError, match="output_size must be <= n"):
        ops.butterfly_multiply_fw(tw, x, True, 9)
    with pytest.raises(RuntimeError, match="must have dimension"):
        ops.butterfly_multiply_fw(tw, x[0], True, None)
    # host tensors run on the operators' own host path (the reference's three operators only) ...
    from butterfly_amd.multiply import butterfly_multiply_torch
    assert torch.allclose(ops.butterfly_multiply_fw(tw, x, True, None), butterfly_multiply_torch(tw, x, True), atol=1e-6)
    # ... the operators that are new here take device tensors and say so, loudly
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.butterfly_multiply_bias_fw(tw, x, torch.randn(1, 8), True, None)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.butterfly_multiply_base4_fw(torch.randn(1, 1, 1, 2, 4, 4), torch.randn(1, 1, 1, 4, 2, 2), x, True, None)
    # the wrappers are TorchScript-callable like the reference's scripted functions
    @torch.jit.script
    def scripted(t: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        return torch.ops.torch_butterfly.butterfly_multiply(t, v, True, None)
    assert torch.equal(scripted(tw, x), ops.butterfly_multiply_fw(tw, x, True, None))


@pytest.mark.parametrize("inc", [True, False])
def test_twiddle_base2_to_base4_host(inc):
    from butterfly_amd.multiply_base4 import butterfly_multiply_base4_torch, twiddle_base2_to_base4
    from butterfly_amd.multiply import butterfly_multiply_torch
    rng = np.random.default_rng(0)
    for L in (1, 2, 3, 4, 5, 6):
        for nb in (1, 2, 3):
            n = 1 << L
            dtype = np.complex128 if L % 2 else np.float64
            tw = randn(rng, (2, nb, L, n // 2, 2, 2), dtype)
            t4, t2 = twiddle_base2_to_base4(torch.from_numpy(tw), inc)
            o4, o2 = oracle.twiddle_base2_to_base4(tw, inc)
            assert t2.shape == o2.shape and rel_err(t4.numpy(), o4) < 1e-12
            if L % 2:
                assert np.array_equal(t2.numpy(), o2)
            x = randn(rng, (3, 2, n - 1 if n > 2 else n), dtype)
            y2 = butterfly_multiply_torch(torch.from_numpy(tw), torch.from_numpy(x), inc)
            y4 = butterfly_multiply_base4_torch(t4, t2, torch.from_numpy(x), inc)
            assert rel_err(y4.numpy(), y2.numpy()) < 1e-12
            assert rel_err(y2.numpy(), oracle.butterfly_fw(tw, x, inc)) < 1e-12
            assert rel_err(y4.numpy(), oracle.butterfly_base4_fw(o4, o2, x, inc)) < 1e-12


def test_torch_restatement_gradients_match_oracle():
    from butterfly_amd.multiply import butterfly_multiply_torch
    from butterfly_amd.multiply_base4 import butterfly_multiply_base4_torch
    rng = np.random.default_rng(1)
    for dtype in (np.float64, np.complex128):
        L, nb, B, S = 5, 2, 4, 2
        n = 1 << L
        tw = randn(rng, (S, nb, L, n // 2, 2, 2), dtype)
        x = randn(rng, (B, S, n - 3), dtype)
        g = randn(rng, (B, S, n - 5), dtype)
        t, xx = torch.from_numpy(tw).requires_grad_(), torch.from_numpy(x).requires_grad_()
        y = butterfly_multiply_torch(t, xx, False, n - 5)
        dt, dx = torch.autograd.grad(y, (t, xx), torch.from_numpy(g))
        dt_ref, dx_ref = oracle.butterfly_bw(tw, x, g, False)
        assert rel_err(dt.numpy(), dt_ref) < 1e-12 and rel_err(dx.numpy(), dx_ref) < 1e-12
        tw4 = randn(rng, (S, nb, L // 2, n // 4, 4, 4), dtype)
        tw2 = randn(rng, (S, nb, L % 2, n // 2, 2, 2), dtype)
        t4, t2 = torch.from_numpy(tw4).requires_grad_(), torch.from_numpy(tw2).requires_grad_()
        y = butterfly_multiply_base4_torch(t4, t2, xx, True, n - 5)
        d4, d2, dx = torch.autograd.grad(y, (t4, t2, xx), torch.from_numpy(g))
        d4_ref, d2_ref, dx_ref = oracle.butterfly_base4_bw(tw4, tw2, x, g, True)
        assert rel_err(d4.numpy(), d4_ref) < 1e-12 and rel_err(d2.numpy(), d2_ref) < 1e-12
        assert rel_err(dx.numpy(), dx_ref) < 1e-12


def test_scale_twiddle_folds_diagonals_into_the_end_factors():
    """diag(out) B diag(in), evaluated by the oracle on twiddles with the diagonals folded in,
    against the oracle's B applied between explicit elementwise products; short diagonals
    leave the remaining entries alone."""
    from butterfly_amd.butterfly import scale_twiddle
    rng = np.random.default_rng(11)
    for dtype in (np.float64, np.complex128):
        for inc in (True, False):
            for nb, L, S in [(1, 1, 1), (1, 1, 2), (1, 3, 2), (2, 4, 1), (3, 2, 2)]:
                n = 1 << L
                tw = randn(rng, (S, nb, L, n // 2, 2, 2), dtype)
                x = randn(rng, (5, S, n), dtype)
                d = randn(rng, (max(1, n - 1),), dtype)
                e = randn(rng, (max(1, S * n - 1),), dtype)
                dfull = np.concatenate([d, np.ones(n - d.size, dtype)])
                efull = np.concatenate([e, np.ones(S * n - e.size, dtype)]).reshape(S, n)
                ref = oracle.butterfly_fw(tw, x * dfull, inc) * efull
                folded = scale_twiddle(torch.from_numpy(tw), inc, torch.from_numpy(d), torch.from_numpy(e))
                assert rel_err(oracle.butterfly_fw(folded.numpy(), x, inc), ref) < 1e-12
                only_in = scale_twiddle(torch.from_numpy(tw), inc, torch.from_numpy(d), None)
                assert rel_err(oracle.butterfly_fw(only_in.numpy(), x, inc), oracle.butterfly_fw(tw, x * dfull, inc)) < 1e-12
                only_out = scale_twiddle(torch.from_numpy(tw), inc, None, torch.from_numpy(e))
                assert rel_err(oracle.butterfly_fw(only_out.numpy(), x, inc), oracle.butterfly_fw(tw, x, inc) * efull) < 1e-12


def apply_cpu(b, x):
    """Evaluate a Butterfly module's matrix on the CPU through the oracle (host-logic check
    of the twiddle a constructor produced; the module's own forward needs the device)."""
    xs = np.broadcast_to(x[:, None, :], (x.shape[0], b.nstacks, x.shape[1]))
    tw = b.twiddle.detach().numpy()
    y = oracle.butterfly_fw(tw, xs.astype(tw.dtype), b.increasing_stride, b.out_size if b.nstacks == 1 else None)
    return y.reshape(x.shape[0], -1)[:, :b.out_size]


def test_special_twiddles_on_the_host():
    import scipy.linalg
    from butterfly_amd import special
    from butterfly_amd.permutation import bitreversal_permutation
    rng = np.random.default_rng(2)
    for n in (2, 16, 128):
        br = bitreversal_permutation(n)
        assert sorted(br) == list(range(n)) and np.array_equal(br[br], np.arange(n))
        x = randn(rng, (3, n), np.complex64)
        for normalized in (False, True):
            f = special.fft(n, normalized=normalized, br_first=True, with_br_perm=False)
            want = np.fft.fft(x, norm="ortho" if normalized else None)
            assert rel_err(apply_cpu(f, x[:, br]), want) < 1e-5
            f = special.fft(n, normalized=normalized, br_first=False, with_br_perm=False)
            assert not f.increasing_stride
            assert rel_err(apply_cpu(f, x)[:, br], want) < 1e-5
            fi = special.ifft(n, normalized=normalized, br_first=True, with_br_perm=False)
            want = np.fft.ifft(x, norm="ortho" if normalized else None)
            assert rel_err(apply_cpu(fi, x[:, br]), want) < 1e-5
        h = special.hadamard(n, normalized=False, increasing_stride=False)
        xr = randn(rng, (3, n), np.float32)
        assert rel_err(apply_cpu(h, xr), xr @ scipy.linalg.hadamard(n).T.astype(np.float32)) < 1e-5
    # circulant with the diagonal folded in: one Butterfly with two blocks
    col = torch.from_numpy(randn(rng, (16,), np.complex64))
    b = special.circulant(col, separate_diagonal=False)
    assert b.nblocks == 2 and b.twiddle.shape == (1, 2, 4, 8, 2, 2)
    x = randn(rng, (3, 16), np.complex64)
    assert rel_err(apply_cpu(b, x), x @ scipy.linalg.circulant(col.numpy()).T) < 1e-5


def test_module_bookkeeping():
    import butterfly_amd as bfa
    torch.manual_seed(0)
    b = bfa.Butterfly(7, 15, nblocks=2)
    assert (b.log_n, b.n, b.nstacks) == (3, 8, 2)
    assert list(b.state_dict().keys()) == ["twiddle", "bias"]
    assert b.twiddle.shape == (2, 2, 3, 4, 2, 2) and b.bias.shape == (15,)
    assert b.twiddle._is_structured
    assert b.bias.abs().max() <= 1 / np.sqrt(7)
    for complex_ in (False, True):
        o = bfa.Butterfly(64, 64, complex=complex_, init="ortho", nblocks=3)
        sv = torch.linalg.svdvals(o.twiddle.detach().reshape(-1, 2, 2))
        assert torch.allclose(sv, torch.ones_like(sv), atol=1e-5)
    e = bfa.Butterfly(16, 16, init="identity", bias=False)
    x = np.random.default_rng(0).standard_normal((2, 16)).astype(np.float32)
    assert np.array_equal(apply_cpu(e, x), x)
    f = bfa.Butterfly(16, 16, complex=True, init="fft_no_br", nblocks=2, bias=False)
    assert torch.equal(f.twiddle[:, 1], torch.eye(2, dtype=torch.complex64).expand(1, 4, 8, 2, 2))
    b4 = bfa.ButterflyBase4(32, 32, nblocks=2)
    assert sorted(b4.state_dict().keys()) == ["bias", "twiddle2", "twiddle4"]
    assert b4.twiddle4.shape == (1, 2, 2, 8, 4, 4) and b4.twiddle2.shape == (1, 2, 1, 16, 2, 2)
    before = b.twiddle.detach().clone()
    with torch.no_grad():
        b *= 2.0
    assert torch.allclose(b.twiddle, before * 2.0 ** (1 / 6))
    with pytest.raises(ValueError):
        bfa.Butterfly(8, 8, init=torch.zeros(3))


def _apply_switches(cross, log_n, inc, x):
    """Two-block butterfly of straight / crossed switches applied with numpy."""
    n = 1 << log_n
    y = x.copy()
    for block in range(2):
        block_inc = inc != (block == 1)
        for idx in range(log_n):
            b = idx if block_inc else log_n - 1 - idx
            bit = 1 << b
            e = np.flatnonzero((np.arange(n) & bit) == 0)
            pair = ((e >> (b + 1)) << b) | (e & (bit - 1))
            swap = cross[block, idx, pair]
            out = y.copy()
            out[e[swap]], out[e[swap] ^ bit] = y[e[swap] ^ bit], y[e[swap]]
            y = out
    return y


def test_permutation_routing_and_helpers_on_the_host():
    """The Benes routing behind perm2butterfly realises every permutation (exhaustive for n = 4,
    random up to n = 256), in both stride orders; the small permutation helpers."""
    import itertools
    from butterfly_amd import permutation
    for inc in (False, True):
        for p in itertools.permutations(range(4)):
            cross = permutation._benes_switches(np.array(p), 2, inc)
            assert np.array_equal(_apply_switches(cross, 2, inc, np.arange(4)), np.array(p))
    rng = np.random.default_rng(0)
    for log_n in range(1, 9):
        for inc in (False, True):
            for _ in range(5):
                p = rng.permutation(1 << log_n)
                cross = permutation._benes_switches(p, log_n, inc)
                assert np.array_equal(_apply_switches(cross, log_n, inc, np.arange(1 << log_n)), p)
    assert np.array_equal(permutation.wavelet_permutation(8), [0, 4, 2, 6, 1, 3, 5, 7])
    assert np.array_equal(permutation.wavelet_permutation(2), [0, 1])
    m = permutation.perm_vec_to_mat(np.array([2, 0, 3, 1]))
    x = np.arange(4) * 10
    assert np.array_equal(m, [[0, 1, 0, 0], [0, 0, 0, 1], [1, 0, 0, 0], [0, 0, 1, 0]])   # M[p[i], i] = 1
    assert np.array_equal(x @ m, x[[2, 0, 3, 1]])
    assert np.array_equal(permutation.perm_vec_to_mat(np.array([2, 0, 3, 1]), left=True) @ x, x[[2, 0, 3, 1]])
    assert np.array_equal(permutation.perm_mat_to_vec(m), [2, 0, 3, 1])
    assert np.array_equal(permutation.perm_mat_to_vec(permutation.perm_vec_to_mat([2, 0, 3, 1], left=True), left=True),
                          [2, 0, 3, 1])
    # four diagonal quadrants (one butterfly factor over the whole matrix), not 2 x 2 blocks on the diagonal
    assert permutation.is_2x2_block_diag(np.kron(np.ones((2, 2)), np.diag([1.0, 2.0, 3.0])))
    assert permutation.is_2x2_block_diag(np.ones((2, 2)))
    assert not permutation.is_2x2_block_diag(np.kron(np.eye(3), np.ones((2, 2))))
    assert not permutation.is_2x2_block_diag(np.ones((4, 4)))
    with pytest.raises(ValueError):
        permutation.perm2butterfly(np.array([0, 0, 1]))


def _parse_plan(lines):
    out = []
    for line in lines:
        kind, *fields = line.split()
        d = {"kind": kind}
        for f in fields:
            k, v = f.split("=")
            d[k] = tuple(int(x) for x in v.split("..")) if ".." in v else int(v)
        out.append(d)
    return out


def test_launch_plans_cover_every_stage_once():
    """bf_describe_plan (host only): for every row length up to 2^24, both dtypes, both stride
    orders, forward and backward, the passes cover the stage list exactly once in order; low
    passes hold whole blocks of the `low` lowest bits (10 for float; for complex64 rows of 2048
    to 65536 the smallest width from 6 up that does not add a span); a span pass works on at most five
    (complex64: six) adjacent bits from bit `low` up in one sweep up, one sweep down or both (a
    complex64 pass holds at most ten stages); the spans tile bits low..L-1."""
    from butterfly_amd import _capi
    for cplx in (0, 1):
        for L in range(1, 25):
            span_max = 6 if cplx else 5
            nspans = (max(L, 10) - 10 + span_max - 1) // span_max
            low = max(6, L - span_max * nspans) if cplx and 10 < L <= 16 else min(L, 10)
            for nb in (1, 2, 3):
                for inc in (True, False):
                    for backward in (False, True):
                        batch = 64 if L < 20 else 3
                        plan = _parse_plan(_capi.describe_plan(cplx, batch, 1, L, nb, inc, backward))
                        key = (cplx, L, nb, inc, backward)
                        assert plan and plan[0]["kind"] != "generic", key
                        bits = []
                        for k in range(nb):
                            up = inc != (k % 2 == 1)
                            bits += list(range(L)) if up else list(range(L - 1, -1, -1))
                        t = 0
                        groups = set()
                        for q in plan:
                            a, b = q["t"]
                            assert a == t and b > a, key
                            t = b
                            stage_bits = bits[a:b]
                            if q["kind"] == "low":
                                assert q["L"] == low and b - a == q["L"] * q["nb"], key
                                assert all(x < low for x in stage_bits), key
                                assert q["chunks"] == (1 << (L - low)), key
                                assert q["nb"] <= (1 if cplx else 2), key
                                assert q["inc"] == int(stage_bits[0] == 0 and q["L"] > 1 or (q["L"] == 1 and inc != ((a // L) % 2 == 1))), key
                            elif q["kind"] == "wide":
                                assert not backward and L in (11, 12) and b - a == L, key
                            elif q["kind"] == "span":
                                lb, h = q["lb"], q["bits"]
                                assert lb >= low and 1 <= h <= span_max and q["tiles"] == (1 << (L - 10)), key
                                assert not cplx or b - a <= 10, key
                                up, down = list(range(lb, lb + h)), list(range(lb + h - 1, lb - 1, -1))
                                assert stage_bits == [up, down, up + down][q["mode"]], key
                                groups.add((lb, h))
                            else:
                                raise AssertionError((key, q))
                        assert t == len(bits), key
                        if groups:
                            covered = sorted(x for lb, h in groups for x in range(lb, lb + h))
                            assert covered == list(range(low, L)), key
    # the configurations the benchmark is quoted on
    assert _capi.describe_plan(0, 16384, 1, 10, 2, False, True) == ["low t=0..20 L=10 nb=2 inc=0 chunks=1"]
    assert [l.split()[0] for l in _capi.describe_plan(0, 32768, 1, 12, 2, True, False)] == ["wide", "wide"]
    assert [l.split()[0] for l in _capi.describe_plan(0, 32768, 1, 12, 2, True, True)] == ["low", "span", "low"]
    assert [l.split()[0] for l in _capi.describe_plan(0, 2048, 1, 13, 1, True, True)] == ["low", "span"]
    assert [l.split()[0] for l in _capi.describe_plan(0, 16, 1, 20, 1, True, False)] == ["low", "span", "span"]
    assert _capi.describe_plan(1, 8192, 1, 12, 1, True, True) == ["low t=0..6 L=6 nb=1 inc=1 chunks=64",
                                                                  "span t=6..12 lb=6 bits=6 mode=0 tiles=4"]


def test_kernels_with_counted_memory_waits_use_no_scratch_memory():
    """The register-resident kernels wait for their LDS-direct row fetches with
    `s_waitcnt vmcnt(N)`, N counted by hand from the kernel's own loads and stores.  A register
    spill would put scratch loads and stores of the compiler's between request and wait and make
    N too large: the build records the compiler's resource-usage remarks, and no such kernel may
    show scratch memory or spills."""
    from butterfly_amd import build
    assert os.path.isfile(build.RESOURCES), "run `python -m butterfly_amd.build` first"
    bad, seen = build.check_kernel_resources()
    assert seen >= 200, seen     # every fast_* / wide_* / fast4* instantiation reports
    assert bad == []
    with open(build.RESOURCES) as f:
        kernels = build.parse_kernel_resources(f.read())
    # 1024 threads per workgroup = 16 wavefronts per compute unit: 128 registers each
    assert max(v["VGPRs"] + v["AGPRs"] for k, v in kernels.items() if any(g in k for g in build.GATED_KERNELS)) <= 128


GOLDEN = os.path.join(ROOT, "tests", "golden", "butterfly_ref_cases.npz")


def test_operators_on_host_tensors_match_the_reference_vectors():
    """Host tensors (float, double, complex64, complex128) run on the operators' own host path:
    every golden case written from the compiled reference, through
    torch.ops.torch_butterfly.butterfly_multiply_fw / _bw and through autograd."""
    import butterfly_amd  # noqa: F401
    ops = torch.ops.torch_butterfly
    d = np.load(GOLDEN)
    ncases = len([k for k in d.files if k.endswith("_meta")])
    seen, exact = set(), 0
    for i in range(ncases):
        tw, x, g = (torch.from_numpy(d[f"c{i}_{k}"]) for k in ("twiddle", "input", "grad"))
        inc, osz = [int(v) for v in d[f"c{i}_meta"]]
        osz = None if osz < 0 else osz
        seen.add(tw.dtype)
        y = ops.butterfly_multiply_fw(tw, x, bool(inc), osz)
        dtw, dx = ops.butterfly_multiply_bw(tw, x, g, bool(inc))
        n = 1 << tw.shape[2]
        assert y.shape == d[f"c{i}_output"].shape and y.stride() == (x.shape[1] * n, n, 1)
        tol_fw, tol_bw = (1e-5, 1e-4) if tw.dtype in (torch.float32, torch.complex64) else (1e-12, 1e-11)
        assert rel_err(y.numpy(), d[f"c{i}_output"]) < tol_fw, i
        assert rel_err(dx.numpy(), d[f"c{i}_d_input"]) < tol_bw, i
        assert rel_err(dtw.numpy(), d[f"c{i}_d_twiddle"]) < tol_bw, i
        exact += int(np.array_equal(y.numpy(), d[f"c{i}_output"]) and np.array_equal(dx.numpy(), d[f"c{i}_d_input"])
                     and np.array_equal(dtw.numpy(), d[f"c{i}_d_twiddle"]))
        twr, xr = tw.clone().requires_grad_(), x.clone().requires_grad_()
        ya = ops.butterfly_multiply(twr, xr, bool(inc), osz)
        a_dtw, a_dx = torch.autograd.grad(ya, (twr, xr), g)
        assert torch.equal(ya.detach(), y) and torch.equal(a_dtw, dtw) and torch.equal(a_dx, dx)
    assert seen == {torch.float32, torch.float64, torch.complex64, torch.complex128}
    assert exact == ncases      # same operations in the same order as the reference: identical bits


@pytest.mark.parametrize("batch,n", [(10, 4096), (300, 512)])
def test_reference_multiply_test_on_cpu(batch, n):
    """The reference's own operator test on the 'cpu' device
    (/root/reference/tests/test_multiply.py:17-59; it skips its large-batch shape there, a smaller
    batch of the same row length stands in): operator against the PyTorch restatement, forward
    and both gradients, real and complex, both stride orders, same tolerances."""
    import math
    from butterfly_amd.multiply import butterfly_multiply, butterfly_multiply_torch
    log_n, nstacks, nblocks = int(math.log2(n)), 2, 3
    torch.manual_seed(n)
    for cplx in (False, True):
        for inc in (True, False):
            dtype = torch.complex64 if cplx else torch.float32
            twiddle = (torch.randn(nstacks, nblocks, log_n, n // 2, 2, 2, dtype=dtype) / math.sqrt(2)).requires_grad_()
            x = torch.randn(batch, nstacks, n, dtype=dtype, requires_grad=True)
            out = butterfly_multiply(twiddle, x, inc)
            out_t = butterfly_multiply_torch(twiddle, x, inc)
            assert torch.allclose(out, out_t, rtol=1e-3, atol=1e-5)
            grad = torch.randn_like(out_t)
            d_tw, d_x = torch.autograd.grad(out, (twiddle, x), grad)
            d_tw_t, d_x_t = torch.autograd.grad(out_t, (twiddle, x), grad)
            assert torch.allclose(d_x, d_x_t, rtol=1e-3, atol=1e-5)
            assert torch.allclose(d_tw, d_tw_t, rtol=1e-3, atol=1e-5)


def test_modules_run_on_host_tensors():
    """Butterfly / ButterflyBase4 / special.fft on the CPU, as the reference's modules do."""
    import butterfly_amd
    from butterfly_amd import special
    from butterfly_amd.multiply import butterfly_multiply_torch
    torch.manual_seed(3)
    layer = butterfly_amd.Butterfly(100, 200, bias=True, nblocks=2)
    x = torch.randn(5, 100, requires_grad=True)
    y = layer(x)
    ref = butterfly_multiply_torch(layer.twiddle, layer.pre_process(x), layer.increasing_stride, None)
    ref = ref.reshape(5, -1)[:, :200] + layer.bias
    assert y.shape == (5, 200) and torch.allclose(y, ref, atol=1e-5)
    y.sum().backward()
    assert layer.twiddle.grad is not None and x.grad is not None and layer.bias.grad is not None
    b4 = butterfly_amd.ButterflyBase4(64, 64, bias=False)
    assert b4(torch.randn(3, 64)).shape == (3, 64)
    f = special.fft(64, normalized=True)
    z = torch.randn(4, 64, dtype=torch.complex64)
    assert torch.allclose(f(z), torch.fft.fft(z, norm="ortho"), atol=1e-5)
    dbl = butterfly_amd.Butterfly(16, 16, bias=False).double()
    assert dbl(torch.randn(2, 16, dtype=torch.float64)).dtype == torch.float64


def _soft_factor_matrix(n, stride, p, q0, q1):
    """Dense matrix of one relaxed permutation factor, entry by entry from its definition:
    inside every group of 2 * stride elements, with weight p the even elements are dealt to the
    first half and the odd ones to the second; then half a is reversed with weight q_a."""
    deal = np.zeros((n, n))
    flip = np.zeros((n, n))
    q = (q0, q1)
    for base in range(0, n, 2 * stride):
        for a in range(2):
            for j in range(stride):
                row = base + a * stride + j
                deal[row, row] += 1 - p
                deal[row, base + 2 * j + a] += p
                flip[row, row] += 1 - q[a]
                flip[row, base + a * stride + stride - 1 - j] += q[a]
    return flip @ deal


@pytest.mark.parametrize("inc", [False, True])
def test_legacy_learnable_permutation(inc):
    """The relaxed permutation product against dense matrices built from the definition of a
    factor (output, gradients of input and probabilities), its hard limits against known
    permutations, and the module's bookkeeping (reference: butterfly/permutation.py,
    butterfly/permutation_multiply.py:18-52)."""
    from butterfly_amd import legacy_permutation as lp
    rng = np.random.default_rng(77 + inc)
    n, B = 32, 5
    m = 5
    prob = rng.uniform(0.05, 0.95, (m - 1, 3))
    order = list(range(1, m)) if inc else list(range(1, m))[::-1]
    dense = np.eye(n)
    for k in order:
        dense = _soft_factor_matrix(n, 1 << k, *prob[k - 1]) @ dense
    x = rng.standard_normal((B, n))
    g = rng.standard_normal((B, n))
    pt = torch.tensor(prob, requires_grad=True)
    xt = torch.tensor(x, requires_grad=True)
    y = lp.permutation_mult(pt, xt, increasing_stride=inc)
    assert np.allclose(y.detach().numpy(), x @ dense.T, atol=1e-12)
    d_p, d_x = torch.autograd.grad(y, (pt, xt), torch.tensor(g))
    assert np.allclose(d_x.numpy(), g @ dense, atol=1e-12)
    eps = 1e-6
    for k, c in [(0, 0), (1, 2), (m - 2, 1)]:
        moved = prob.copy()
        moved[k, c] += eps
        dense2 = np.eye(n)
        for kk in order:
            dense2 = _soft_factor_matrix(n, 1 << kk, *moved[kk - 1]) @ dense2
        fd = np.sum(g * (x @ (dense2 - dense).T)) / eps
        assert abs(d_p[k, c].item() - fd) < 1e-4 * max(1.0, abs(fd))
    # complex rows are pairs moved together; intermediates start at the input and end at the output
    xc = torch.tensor(rng.standard_normal((B, n, 2)))
    yc = lp.permutation_mult(pt.detach(), xc, increasing_stride=inc, return_intermediates=True)
    assert yc.shape == (m, B, n, 2) and torch.equal(yc[0], xc)
    for part in range(2):
        assert np.allclose(yc[-1][..., part].numpy(), xc[..., part].numpy() @ dense.T, atol=1e-12)
    # hard limits: dealing inside a group of 2^b elements reads position p from p with its low b bits
    # rotated left by one; widest group first, the rotations compose to the bit reversal
    hard = torch.zeros(m - 1, 3, dtype=torch.float64)
    hard[:, 0] = 1
    idx = torch.arange(n, dtype=torch.float64).unsqueeze(0)

    def rotl(p, b):
        low = p & ((1 << b) - 1)
        return (p - low) | ((low << 1) & ((1 << b) - 1)) | (low >> (b - 1))
    want = []
    for p in range(n):
        src = p
        for b in (range(2, m + 1) if not inc else range(m, 1, -1)):   # last applied factor first
            src = rotl(src, b)
        want.append(src)
    if not inc:
        assert want == [int(format(i, f"0{m}b")[::-1], 2) for i in range(n)]
    assert lp.permutation_mult(hard, idx, increasing_stride=inc).squeeze(0).long().tolist() == want
    # one factor over the whole row: reverse the second half only
    out = lp.permutation_mult_single(torch.tensor([0.0, 0.0, 1.0], dtype=torch.float64), idx).squeeze(0).long().tolist()
    assert out == list(range(n // 2)) + list(range(n - 1, n // 2 - 1, -1))
    # modules
    torch.manual_seed(5)
    for share in (False, True):
        mod = lp.Permutation(n, share_logit=share, increasing_stride=inc)
        assert tuple(mod.logit.shape) == ((3,) if share else (m - 1, 3))
        with torch.no_grad():
            mod.logit.copy_(torch.where(mod.logit > 0, 30.0, -30.0))   # saturated: a permutation up to 1e-12
        p = mod.argmax()
        assert sorted(p.tolist()) == list(range(n))
        xr = torch.randn(B, n)
        assert torch.allclose(mod(xr), lp.FixedPermutation(p)(xr), atol=1e-5)
        assert torch.allclose(mod(xr), xr[:, p], atol=1e-5)
    fac = lp.PermutationFactor(n)
    with torch.no_grad():
        fac.logit.copy_(torch.tensor([30.0, -30.0, 30.0]))
    assert torch.allclose(fac(xr), xr[:, fac.argmax()], atol=1e-5)
    assert fac.argmax().tolist() == list(range(0, n, 2)) + list(range(n - 1, 0, -2))
    with pytest.raises(ValueError):
        lp.Permutation(24)
    with pytest.raises(ValueError):
        lp.permutation_mult(torch.rand(5, 3), torch.randn(2, 32))


def test_permutation_factorisation_following_the_existence_proof():
    """half_balance / modular_balance / modular_balanced_to_butterfly_factor /
    perm2butterfly_slow / outer_twiddle_factors: the properties the reference's own tests state
    (tests/test_permutation.py:34-67), which define these functions up to the free choice inside
    every loop of swaps."""
    import butterfly_amd
    from butterfly_amd import permutation as P
    rng = np.random.default_rng(21)
    for n in (2, 4, 16, 64, 256):
        for _ in range(10):
            v = rng.permutation(n)
            perm, balanced = P.half_balance(v)
            assert np.array_equal(balanced, v[perm]) and np.array_equal(perm[perm], np.arange(n))
            assert np.all(np.abs(perm - np.arange(n)) % (n // 2) == 0)           # only i <-> i + n/2
            for half in (balanced[:n // 2], balanced[n // 2:]):
                assert np.array_equal(np.sort(half % (n // 2)), np.arange(n // 2))
            low, balanced2 = P.half_balance(v, return_swap_locations=True)
            assert np.array_equal(balanced2, balanced) and sorted(low) == list(np.flatnonzero(perm[:n // 2] != np.arange(n // 2)))
            perms, w = P.modular_balance(v)
            assert len(perms) == n.bit_length() - 1 and P.is_modular_balanced(w)
            assert P.is_modular_balanced(P.perm_vec_to_mat(w))
            v2 = v
            for p in perms:
                v2 = v2[p]
            assert np.array_equal(v2, w)
            back = w
            for p in reversed(perms):
                back = back[P.invert(p)]
            assert np.array_equal(back, v)
            mat = P.perm_vec_to_mat(v)
            for p in perms:                                   # x M_v M_p = x[v][p]
                mat = mat @ P.perm_vec_to_mat(p)
            assert np.array_equal(mat, P.perm_vec_to_mat(w))
            factors = P.modular_balanced_to_butterfly_factor(w)
            prod = np.eye(n, dtype=np.int64)
            for i, f in enumerate(factors):
                assert P.is_butterfly_factor(f, n >> i)
                prod = prod @ f
            assert np.array_equal(prod, P.perm_vec_to_mat(w))
            assert all(np.array_equal(a, b) for a, b in
                       zip(factors, P.modular_balanced_to_butterfly_factor(P.perm_vec_to_mat(w))))
    assert not P.is_modular_balanced(np.array([0, 2, 1, 3]))
    assert P.is_modular_balanced(np.array([0, 1, 2, 3])) and P.is_modular_balanced(np.array([3, 0, 1, 2]))
    with pytest.raises(ValueError):
        P.modular_balanced_to_butterfly_factor(np.array([0, 2, 1, 3]))
    for n in (2, 13, 38):
        for inc in (False, True):
            for cplx in (False, True):
                for _ in range(5):
                    v = torch.from_numpy(rng.permutation(n))
                    b = P.perm2butterfly_slow(v, cplx, inc)
                    assert (b.in_size, b.out_size, b.nblocks, b.increasing_stride) == (n, n, 2, inc)
                    x = torch.arange(n, dtype=torch.float32).to(torch.complex64 if cplx else torch.float32)
                    assert torch.equal(b(x), x[v])
    # the level-by-level recursion: first switch column, last switch column, two half-size problems
    for log_n in (1, 3, 6):
        n = 1 << log_n
        v = rng.permutation(n)
        cur = v[None]
        first, last = [], []
        for level in range(log_n):
            f, l, cur = P.outer_twiddle_factors(cur)
            assert f.shape == l.shape == (n // 2, 2, 2) and cur.shape == (2 << level, n >> (level + 1))
            first.append(f)
            last.append(l)
        twiddle = torch.stack([torch.stack(first), torch.stack(last).flip([0])]).unsqueeze(0)
        b = butterfly_amd.Butterfly(n, n, bias=False, increasing_stride=False, init=twiddle, nblocks=2)
        x = torch.arange(n, dtype=torch.float32)
        assert torch.equal(b(x), x[torch.from_numpy(v)])
    v = torch.from_numpy(rng.permutation(11))
    x = torch.randn(3, 11)
    assert torch.equal(P.FixedPermutation(v).to_butterfly(increasing_stride=True)(x), x[:, v])
    t = P.swap_locations_to_twiddle_factor(8, [1, 3])
    assert t.shape == (4, 2, 2) and torch.equal(t[0], torch.eye(2)) and torch.equal(t[1], torch.tensor([[0.0, 1.0], [1.0, 0.0]]))


def test_complex_helpers():
    """complex_matmul and index_last_dim as the reference's tests/test_complex_utils.py checks them
    (against broadcast-multiply-and-sum, gradients included), the four-real-products form, and
    ComplexLinear against the product written out."""
    from butterfly_amd import complex_utils as cu
    torch.manual_seed(3)
    X = torch.randn(3, 5, 64, 16, dtype=torch.complex64, requires_grad=True)
    Y = torch.randn(3, 5, 16, 32, dtype=torch.complex64, requires_grad=True)
    want = (X.unsqueeze(-1) * Y.unsqueeze(-3)).sum(dim=-2)
    g = torch.randn_like(want)
    for product in (cu.complex_matmul, cu.complex_matmul_torch):
        got = product(X, Y)
        assert torch.allclose(got, want, 1e-3, 1e-5)
        for a, b in zip(torch.autograd.grad(got, (X, Y), g), torch.autograd.grad(want, (X, Y), g, retain_graph=True)):
            assert torch.allclose(a, b, 1e-3, 1e-4)
    p = torch.randperm(17)
    x = torch.randn(2, 3, 17, requires_grad=True)
    out = cu.index_last_dim(x, p)
    gg = torch.randn_like(out)
    assert torch.equal(out, x[..., p])
    assert torch.equal(torch.autograd.grad(out, x, gg)[0], torch.autograd.grad(x[..., p], x, gg)[0])
    assert cu.IndexLastDim.apply(x, p).equal(out) and cu.Real2ComplexFn.apply(x).dtype == torch.complex64
    lin = cu.ComplexLinear(12, 7)
    assert lin.weight.shape == (7, 12) and lin.weight.dtype == torch.complex64 and lin.bias.shape == (7,)
    assert lin.weight.abs().max() <= 1 / 12 ** 0.5 + 1e-6
    z = torch.randn(4, 5, 12, dtype=torch.complex64)
    assert torch.allclose(lin(z), (z.unsqueeze(-2) * lin.weight).sum(-1) + lin.bias, 1e-4, 1e-5)
    assert cu.ComplexLinear(12, 7, bias=False).bias is None


def test_legacy_plain_pytorch_twins_and_dyadic_multiply():
    """The legacy package's `*_torch` names and `butterfly_mult_dyadic_torch` (factors with
    arbitrary strides in the order given), on host tensors, against the numpy restatement's
    single-factor step applied literally, intermediates included."""
    from butterfly_amd import legacy
    from oracle import legacy_oracle as lo
    rng = np.random.default_rng(31)
    n, m, S, B = 16, 4, 2, 5
    for cplx in (False, True):
        def to_t(a):
            return torch.from_numpy(np.stack((a.real, a.imag), -1).astype(np.float32)) if cplx else torch.from_numpy(a.astype(np.float32))

        def to_n(t):
            a = t.detach().numpy().astype(np.float64)
            return a[..., 0] + 1j * a[..., 1] if cplx else a

        def rnd(shape):
            a = rng.standard_normal(shape)
            return a + 1j * rng.standard_normal(shape) if cplx else a
        x = rnd((B, S, n))
        strides = [2, 0, 3, 3, 1]
        tw = rnd((S, len(strides), n // 2, 2, 2)) / np.sqrt(2)
        steps = legacy.butterfly_mult_dyadic_torch(to_t(tw), to_t(x), strides, return_intermediates=True)
        value = x
        assert rel_err(to_n(steps[0]), value) < 1e-6
        for i, ls in enumerate(strides):
            value = lo.factor_apply(tw[:, i], ls, value)
            assert rel_err(to_n(steps[i + 1]), value) < 1e-5
        assert rel_err(to_n(legacy.butterfly_mult_dyadic_torch(to_t(tw), to_t(x), strides)), value) < 1e-5
        for inc in (True, False):
            untied = rnd((S, m, n // 2, 2, 2)) / np.sqrt(2)
            y_ref = lo.butterfly_mult_untied(untied, x, inc)
            assert rel_err(to_n(legacy.butterfly_mult_untied_torch(to_t(untied), to_t(x), inc)), y_ref) < 1e-5
            trail = legacy.butterfly_mult_untied_torch(to_t(untied), to_t(x), inc, return_intermediates=True)
            assert trail.shape[0] == m + 1 and rel_err(to_n(trail[-1]), y_ref) < 1e-5
            value = x
            for i, ls in enumerate(range(m) if inc else range(m - 1, -1, -1)):
                value = lo.factor_apply(untied[:, ls], ls, value)
                assert rel_err(to_n(trail[i + 1]), value) < 1e-5
            tied = rnd((S, n - 1, 2, 2)) / np.sqrt(2)
            y_ref = lo.butterfly_mult(tied, x, inc)
            assert rel_err(to_n(legacy.butterfly_mult_torch(to_t(tied), to_t(x), inc)), y_ref) < 1e-5
            assert rel_err(to_n(legacy.butterfly_mult_torch(to_t(tied), to_t(x), inc, True)[-1]), y_ref) < 1e-5
    bbt = rng.standard_normal((S, 2 * m, n // 2, 2, 2)) / np.sqrt(2)
    xr = rng.standard_normal((B, S, n))
    got = legacy.bbt_mult_untied_torch(torch.from_numpy(bbt).float(), torch.from_numpy(xr).float())
    assert rel_err(got.numpy().astype(np.float64), lo.bbt_mult_untied(bbt, xr)) < 1e-5
    assert legacy.butterfly_ortho_mult_tied_torch is legacy.butterfly_ortho_mult_tied
    with pytest.raises(ValueError):
        legacy.butterfly_mult_dyadic_torch(torch.zeros(S, 2, n // 2, 2, 2), torch.zeros(B, S, n), [0, 1, 2])


def test_legacy_pair_helpers():
    from butterfly_amd import legacy
    torch.manual_seed(2)
    a, b = torch.randn(3, 4, 5, 2), torch.randn(3, 5, 6, 2)
    ac, bc = torch.view_as_complex(a), torch.view_as_complex(b)
    assert torch.allclose(torch.view_as_complex(legacy.complex_matmul(a, b)), ac @ bc, atol=1e-5)
    assert torch.allclose(torch.view_as_complex(legacy.complex_mul(a[:, :, :1], a)), ac[:, :, :1] * ac, atol=1e-6)
    assert torch.equal(legacy.conjugate(a), a * torch.tensor([1.0, -1.0]))
    assert torch.equal(legacy.real_to_complex(a[..., 0])[..., 1], torch.zeros(3, 4, 5))
    assert legacy.bitreversal_permutation(8).tolist() == [0, 4, 2, 6, 1, 5, 3, 7]


def test_layers_of_size_one():
    """in_size = 1 is n = 1, log n = 0: no factors at all, every stack copies its input and adds
    its bias.  (The bias used to be laid out over 2 * (n / 2) = 0 columns there.)"""
    import butterfly_amd
    torch.manual_seed(0)
    x = torch.randn(4, 1)
    b = butterfly_amd.Butterfly(1, 5, bias=True)
    assert b.twiddle.numel() == 0 and b.nstacks == 5
    assert torch.allclose(b(x), x.expand(4, 5) + b.bias)
    bmm = butterfly_amd.ButterflyBmm(1, 5, 3, bias=True, nblocks=2)
    xs = torch.randn(4, 3, 1)
    assert torch.allclose(bmm(xs), xs.expand(4, 3, 5) + bmm.bias)
    g = torch.autograd.grad(bmm(xs).sum(), bmm.bias)[0]
    assert torch.equal(g, torch.full_like(g, 4.0))


def test_permuted_multiply_of_size_one_on_the_host():
    """The host form of butterfly_multiply_perm at n = 1 (log n = 0, no pairs) with a column
    table: one column in, one column out, the bias added."""
    from butterfly_amd.multiply import butterfly_multiply_perm
    tw = torch.zeros(3, 2, 0, 0, 2, 2)
    x = torch.randn(4, 3, 1)
    table = torch.zeros(1, dtype=torch.int32)
    bias = torch.randn(3, 1)
    y = butterfly_multiply_perm(tw, x, table, table, bias, True, None)
    assert y.shape == (4, 3, 1) and torch.allclose(y, x + bias)
    assert torch.allclose(butterfly_multiply_perm(tw, x, None, None, None, False, 1), x)
