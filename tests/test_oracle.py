"""Pins the CPU oracle: golden vectors from the compiled reference, the live reference build
where present, closed forms, dense brute force and adjoint / finite-difference identities."""
import os
import subprocess
import sys

import numpy as np
import pytest
import scipy.linalg

from conftest import ROOT, dense_butterfly, dense_stage2, dense_stage4, randn, rel_err
from oracle import oracle

GOLDEN = os.path.join(ROOT, "tests", "golden", "butterfly_ref_cases.npz")
REF_SO = os.path.join(ROOT, "oracle", "_ref", "_butterfly_ref.so")
DTYPES = [np.float32, np.float64, np.complex64, np.complex128]


def test_golden_vectors_bit_exact():
    d = np.load(GOLDEN)
    ncases = len([k for k in d.files if k.endswith("_meta")])
    assert ncases >= 50
    for i in range(ncases):
        tw, x, g = d[f"c{i}_twiddle"], d[f"c{i}_input"], d[f"c{i}_grad"]
        inc, osz = [int(v) for v in d[f"c{i}_meta"]]
        y = oracle.butterfly_fw(tw, x, bool(inc), None if osz < 0 else osz)
        dtw, dx = oracle.butterfly_bw(tw, x, g, bool(inc))
        assert np.array_equal(y, d[f"c{i}_output"]), i
        assert np.array_equal(dtw, d[f"c{i}_d_twiddle"]), i
        assert np.array_equal(dx, d[f"c{i}_d_input"]), i


@pytest.mark.skipif(not os.path.isfile(REF_SO), reason="reference build (oracle/_ref) not present")
def test_live_reference_bit_exact(tmp_path):
    """Fresh seeds and larger sizes than the committed vectors, against the compiled reference."""
    rng = np.random.default_rng(7)
    cases = [(np.float32, 5, 2, 9, 3, 512, -1, 1), (np.float32, 3, 1, 10, 2, 1024, -1, 0),
             (np.complex64, 3, 2, 8, 3, 256, -1, 0), (np.float64, 2, 1, 6, 4, 50, 33, 1),
             (np.complex128, 2, 2, 5, 1, 70, 20, 0), (np.float32, 40, 1, 7, 2, 128, 128, 1)]
    blob = {}
    for i, (dt, B, S, L, nb, I, O, inc) in enumerate(cases):
        n = 1 << L
        blob[f"c{i}_twiddle"] = (randn(rng, (S, nb, L, n // 2, 2, 2), dt) / np.sqrt(2)).astype(dt)
        blob[f"c{i}_input"] = randn(rng, (B, S, I), dt)
        blob[f"c{i}_grad"] = randn(rng, (B, S, n if O < 0 else O), dt)
        blob[f"c{i}_meta"] = np.array([inc, O], dtype=np.int64)
    fin, fout = str(tmp_path / "in.npz"), str(tmp_path / "out.npz")
    np.savez(fin, **blob)
    subprocess.check_call([sys.executable, os.path.join(ROOT, "oracle", "ref_runner.py"), "run", fin, fout])
    res = np.load(fout)
    for i, (dt, B, S, L, nb, I, O, inc) in enumerate(cases):
        y = oracle.butterfly_fw(blob[f"c{i}_twiddle"], blob[f"c{i}_input"], bool(inc), None if O < 0 else O)
        dtw, dx = oracle.butterfly_bw(blob[f"c{i}_twiddle"], blob[f"c{i}_input"], blob[f"c{i}_grad"], bool(inc))
        assert np.array_equal(y, res[f"c{i}_output"])
        assert np.array_equal(dtw, res[f"c{i}_d_twiddle"])
        assert np.array_equal(dx, res[f"c{i}_d_input"])


@pytest.mark.parametrize("inc", [True, False])
def test_identity_and_hadamard_closed_forms(inc):
    rng = np.random.default_rng(0)
    for L in range(1, 8):
        n = 1 << L
        x = randn(rng, (3, 1, n), np.float64)
        eye = np.broadcast_to(np.eye(2), (1, 1, L, n // 2, 2, 2)).copy()
        assert np.array_equal(oracle.butterfly_fw(eye, x, inc), x)
        had = np.broadcast_to(np.array([[1.0, 1.0], [1.0, -1.0]]), (1, 1, L, n // 2, 2, 2)).copy()
        y = oracle.butterfly_fw(had, x, inc)
        np.testing.assert_allclose(y[:, 0], x[:, 0] @ scipy.linalg.hadamard(n).T, rtol=1e-12, atol=1e-12)


def test_fft_closed_form():
    """Cooley-Tukey factors + bit reversal reproduce numpy's FFT (formula stated independently)."""
    rng = np.random.default_rng(1)
    for L in range(1, 9):
        n = 1 << L
        tw = np.zeros((1, 1, L, n // 2, 2, 2), dtype=np.complex128)
        for idx in range(L):
            size = 2 << idx
            for i in range(n // 2):
                w = np.exp(-2j * np.pi * (i % (size // 2)) / size)
                tw[0, 0, idx, i] = [[1, w], [1, -w]]
        br = np.array([int(format(i, f"0{L}b")[::-1], 2) for i in range(n)])
        x = randn(rng, (4, 1, n), np.complex128)
        y = oracle.butterfly_fw(tw, x[:, :, br], True)
        np.testing.assert_allclose(y, np.fft.fft(x, axis=-1), rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inc", [True, False])
def test_dense_brute_force(dtype, inc):
    rng = np.random.default_rng(2)
    tol = 1e-5 if np.dtype(dtype).itemsize in (4, 8) and np.dtype(dtype) in (np.float32, np.complex64) else 1e-12
    for L, nb in [(1, 1), (2, 3), (4, 2), (6, 3)]:
        n = 1 << L
        tw = (randn(rng, (2, nb, L, n // 2, 2, 2), dtype) / np.sqrt(2)).astype(dtype)
        for I, O in [(n, None), (n - 3 if n > 4 else n, n // 2), (2 * n + 1, None)]:
            x = randn(rng, (3, 2, I), dtype)
            xp = np.zeros((3, 2, n), dtype=dtype)
            xp[:, :, :min(I, n)] = x[:, :, :n]
            y = oracle.butterfly_fw(tw, x, inc, O)
            for s in range(2):
                M = dense_butterfly(tw[s].astype(np.complex128), inc)
                want = (xp[:, s].astype(np.complex128) @ M.T)[:, :O]
                assert rel_err(y[:, s], want.astype(dtype) if np.dtype(dtype).kind == 'c' else want.real.astype(dtype)) < tol


@pytest.mark.parametrize("dtype", [np.float64, np.complex128])
@pytest.mark.parametrize("inc", [True, False])
def test_backward_is_the_adjoint_and_matches_dense_gradient(dtype, inc):
    """d_input = M^H g; d_twiddle from the dense formula: for stage k,
    dT = sum_b (A_k^H g)_r conj((B_k x)_c) with A_k the stages after k and B_k those before."""
    rng = np.random.default_rng(3)
    L, nb, B, S = 4, 3, 5, 2
    n = 1 << L
    I, O = n - 2, n - 3
    tw = randn(rng, (S, nb, L, n // 2, 2, 2), dtype)
    x = randn(rng, (B, S, I), dtype)
    g = randn(rng, (B, S, O), dtype)
    dtw, dx = oracle.butterfly_bw(tw, x, g, inc)
    xp = np.zeros((B, S, n), dtype=dtype); xp[:, :, :I] = x
    gp = np.zeros((B, S, n), dtype=dtype); gp[:, :, :O] = g
    for s in range(S):
        stages = []
        for block in range(nb):
            cur = bool(inc) != bool(block % 2)
            for idx in range(L):
                ls = idx if cur else L - 1 - idx
                stages.append((block, idx, ls, dense_stage2(n, ls, tw[s, block, idx])))
        M = np.eye(n, dtype=dtype)
        for *_, Mk in stages:
            M = Mk @ M
        np.testing.assert_allclose(dx[:, s], (gp[:, s] @ M.conj())[:, :I], rtol=1e-10, atol=1e-10)
        for k, (block, idx, ls, _) in enumerate(stages):
            before = np.eye(n, dtype=dtype)
            for *_, Mk in stages[:k]:
                before = Mk @ before
            after = np.eye(n, dtype=dtype)
            for *_, Mk in stages[k + 1:]:
                after = Mk @ after
            xin = xp[:, s] @ before.T            # input of stage k
            gout = gp[:, s] @ after.conj()       # gradient w.r.t. output of stage k
            st = 1 << ls
            for i in range(n // 2):
                low = i % st
                pos = 2 * (i - low) + low
                for r in range(2):
                    for c in range(2):
                        want = np.sum(gout[:, pos + r * st] * np.conj(xin[:, pos + c * st]))
                        assert abs(dtw[s, block, idx, i, r, c] - want) < 1e-9 * max(1, abs(want))


def test_backward_finite_differences():
    rng = np.random.default_rng(4)
    L, nb, B, S = 3, 2, 4, 1
    n = 1 << L
    tw = randn(rng, (S, nb, L, n // 2, 2, 2), np.float64)
    x = randn(rng, (B, S, n), np.float64)
    g = randn(rng, (B, S, n), np.float64)
    dtw, dx = oracle.butterfly_bw(tw, x, g, False)
    eps = 1e-6
    loss = lambda t, xx: float(np.sum(oracle.butterfly_fw(t, xx, False) * g))
    flat = tw.reshape(-1)
    for j in rng.choice(flat.size, 12, replace=False):
        tp, tm = flat.copy(), flat.copy()
        tp[j] += eps; tm[j] -= eps
        fd = (loss(tp.reshape(tw.shape), x) - loss(tm.reshape(tw.shape), x)) / (2 * eps)
        assert abs(fd - dtw.reshape(-1)[j]) < 1e-6
    for j in rng.choice(x.size, 8, replace=False):
        xp_, xm_ = x.reshape(-1).copy(), x.reshape(-1).copy()
        xp_[j] += eps; xm_[j] -= eps
        fd = (loss(tw, xp_.reshape(x.shape)) - loss(tw, xm_.reshape(x.shape))) / (2 * eps)
        assert abs(fd - dx.reshape(-1)[j]) < 1e-6


# ---- base-4 -----------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [np.float64, np.complex128, np.float32])
@pytest.mark.parametrize("inc", [True, False])
def test_base4_dense_brute_force(dtype, inc):
    rng = np.random.default_rng(5)
    for L, nb in [(2, 1), (3, 2), (4, 3), (5, 2), (6, 1)]:
        n = 1 << L
        S, B = 2, 3
        tw4 = randn(rng, (S, nb, L // 2, n // 4, 4, 4), dtype)
        tw2 = randn(rng, (S, nb, L % 2, n // 2, 2, 2), dtype)
        x = randn(rng, (B, S, n - 1), dtype)
        xp = np.zeros((B, S, n), dtype=dtype); xp[:, :, :n - 1] = x
        y = oracle.butterfly_base4_fw(tw4, tw2, x, inc, n - 2)
        for s in range(S):
            M = np.eye(n, dtype=np.complex128)
            for block in range(nb):
                cur = bool(inc) != bool(block % 2)
                for idx in range(L // 2):
                    ls = 2 * idx if cur else L - 2 - 2 * idx
                    M = dense_stage4(n, ls, tw4[s, block, idx].astype(np.complex128)) @ M
                if L % 2:
                    M = dense_stage2(n, L - 1 if cur else 0, tw2[s, block, 0].astype(np.complex128)) @ M
            want = (xp[:, s].astype(np.complex128) @ M.T)[:, :n - 2]
            want = want if np.dtype(dtype).kind == 'c' else want.real
            assert rel_err(y[:, s], want.astype(dtype)) < (1e-5 if dtype == np.float32 else 1e-12)


@pytest.mark.parametrize("inc", [True, False])
def test_base4_equals_base2_after_fusion(inc):
    """tests/test_multiply_base4.py:21-44 of the reference: n = 2..1024, nblocks = 1..4."""
    rng = np.random.default_rng(6)
    for L in range(1, 11):
        for nb in ([1, 2, 3, 4] if L <= 6 else [2]):
            n = 1 << L
            dtype = np.complex128 if L % 2 else np.float64
            tw = randn(rng, (2, nb, L, n // 2, 2, 2), dtype)
            x = randn(rng, (2, 2, n), dtype)
            tw4, tw2 = oracle.twiddle_base2_to_base4(tw, inc)
            y4 = oracle.butterfly_base4_fw(tw4, tw2, x, inc)
            y2 = oracle.butterfly_fw(tw, x, inc)
            assert rel_err(y4, y2) < 1e-12, (L, nb)


@pytest.mark.parametrize("dtype", [np.float64, np.complex128])
def test_base4_backward_adjoint_and_finite_differences(dtype):
    rng = np.random.default_rng(8)
    for L, inc in [(4, True), (5, False), (3, True)]:
        n = 1 << L
        S, B, nb = 2, 3, 2
        tw4 = randn(rng, (S, nb, L // 2, n // 4, 4, 4), dtype)
        tw2 = randn(rng, (S, nb, L % 2, n // 2, 2, 2), dtype)
        x = randn(rng, (B, S, n + 3), dtype)
        g = randn(rng, (B, S, n - 1), dtype)
        d4, d2, dx = oracle.butterfly_base4_bw(tw4, tw2, x, g, inc)
        assert dx.shape == x.shape and np.all(dx[:, :, n:] == 0)
        y = oracle.butterfly_base4_fw(tw4, tw2, x, inc, n - 1)
        # <y(x), g> is real-linear in x: directional derivative equals Re<dx, h>
        h = randn(rng, x.shape, dtype)
        yh = oracle.butterfly_base4_fw(tw4, tw2, x + h, inc, n - 1)
        lhs = np.sum((yh - y) * np.conj(g)).real
        rhs = np.sum(h * np.conj(dx)).real
        assert abs(lhs - rhs) < 1e-9 * max(1.0, abs(lhs))
        # twiddle directions (the map is linear in each single factor entry)
        for tw, d, which in ((tw4, d4, 0), (tw2, d2, 1)):
            if tw.size == 0:
                continue
            for j in rng.choice(tw.size, 6, replace=False):
                e = np.zeros(tw.size, dtype=dtype); e[j] = 1.0
                e = e.reshape(tw.shape)
                args = (tw4 + e, tw2) if which == 0 else (tw4, tw2 + e)
                ye = oracle.butterfly_base4_fw(*args, x, inc, n - 1)
                lhs = np.sum((ye - y) * np.conj(g))
                # d = sum g conj(dy/dt)  =>  sum dy conj(g) = conj(d)
                assert abs(lhs - np.conj(d.reshape(-1)[j])) < 1e-8 * max(1.0, abs(lhs))


# ---- legacy package oracle (oracle/legacy_oracle.py) ---------------------------------------------

from oracle import legacy_oracle as lo  # noqa: E402


def _rand(rng, shape, cplx):
    a = rng.standard_normal(shape)
    return a + 1j * rng.standard_normal(shape) if cplx else a


@pytest.mark.parametrize("cplx", [False, True])
def test_legacy_factor_against_dense_matrix(cplx):
    """Each factor equals the n x n matrix written entry by entry from the pairing rule."""
    rng = np.random.default_rng(11)
    S, n, B = 2, 16, 3
    for ls in range(4):
        st = 1 << ls
        T = _rand(rng, (S, n // 2, 2, 2), cplx)
        x = _rand(rng, (B, S, n), cplx)
        y = lo.factor_apply(T, ls, x)
        for s in range(S):
            M = np.zeros((n, n), dtype=T.dtype)
            for i in range(n // 2):
                low = i % st
                p = (2 * (i // st) * st + low, 2 * (i // st) * st + low + st)
                for r in range(2):
                    for c in range(2):
                        M[p[r], p[c]] = T[s, i, r, c]
            assert np.allclose(y[:, s], x[:, s] @ M.T, rtol=1e-12, atol=1e-12)


def _bitrev(n):
    m = n.bit_length() - 1
    return np.array([int(format(i, f"0{m}b")[::-1], 2) for i in range(n)])


def test_legacy_tied_and_untied_products_are_the_fft():
    """Decimation in time: increasing stride on bit-reversed input with [[1, w], [1, -w]];
    decimation in frequency: decreasing stride with [[1, 1], [w, -w]] and bit-reversed output.
    Neither 2x2 is symmetric and w depends on the position inside the group."""
    rng = np.random.default_rng(12)
    n, B = 32, 4
    x = _rand(rng, (B, 1, n), True)
    ref = np.fft.fft(x, axis=-1)
    br = _bitrev(n)
    tied_dit = np.zeros((1, n - 1, 2, 2), dtype=complex)
    tied_dif = np.zeros((1, n - 1, 2, 2), dtype=complex)
    for ls in range(5):
        st = 1 << ls
        for low in range(st):
            w = np.exp(-2j * np.pi * low / (2 * st))
            tied_dit[0, st - 1 + low] = [[1, w], [1, -w]]
            tied_dif[0, st - 1 + low] = [[1, 1], [w, -w]]
    assert np.allclose(lo.butterfly_mult(tied_dit, x[..., br], True), ref)
    assert np.allclose(lo.butterfly_mult(tied_dif, x, False)[..., br], ref)
    untied = np.stack([lo.tied_expand(tied_dit, ls, n) for ls in range(5)], axis=1)
    assert np.allclose(lo.butterfly_mult_untied(untied, x[..., br], True), ref)
    untied = np.stack([lo.tied_expand(tied_dif, ls, n) for ls in range(5)], axis=1)
    assert np.allclose(lo.butterfly_mult_untied(untied, x, False)[..., br], ref)


def test_legacy_rotation_sign_and_orthogonality():
    theta = np.array([[0.3]])
    x = np.array([[[2.0, 5.0]]])
    y = lo.butterfly_ortho_mult_tied(theta, x, True)
    c, s = np.cos(0.3), np.sin(0.3)
    assert np.allclose(y[0, 0], [c * 2 - s * 5, s * 2 + c * 5])
    rng = np.random.default_rng(13)
    n, m, S = 16, 4, 2
    x = rng.standard_normal((5, S, n))
    norm = np.linalg.norm(x, axis=-1)
    th = rng.uniform(0, 2 * np.pi, (S, 3 * 2 * m, n // 2))
    assert np.allclose(np.linalg.norm(lo.bbt_ortho_mult_untied(th, x), axis=-1), norm)
    assert np.allclose(np.linalg.norm(lo.odo_mult_untied(th, np.ones((S, 3, n)), x), axis=-1), norm)
    tht = rng.uniform(0, 2 * np.pi, (S, 4, n - 1))
    assert np.allclose(np.linalg.norm(lo.bbt_ortho_mult_tied(tht, x), axis=-1), norm)
    # one block, unit diagonal: the ODO product is the B B^T product of the same angles
    assert np.allclose(lo.odo_mult_untied(th[:, :2 * m], np.ones((S, 1, n)), x), lo.bbt_ortho_mult_untied(th[:, :2 * m], x))
    # and the diagonal sits between the two halves
    d = rng.standard_normal((S, 1, n))
    half = lo.butterfly_ortho_mult_untied(th[:, :m][:, ::-1], x, False)
    assert np.allclose(lo.odo_mult_untied(th[:, :2 * m], d, x), lo.butterfly_ortho_mult_untied(th[:, m:2 * m], half * d[:, 0], True))


def test_legacy_fast_format_element_formula():
    """The converter restated operation by operation against the element formula: position e of
    the stride-2^i slice holds T[pair(e)][r][r] (plane 0) and T[pair(e)][r][1 - r] (plane 1),
    r = bit i of e."""
    rng = np.random.default_rng(14)
    S, m = 2, 4
    n = 1 << m
    tw = rng.standard_normal((S, m, n // 2, 2, 2))
    fast = lo.twiddle_normal_to_fast_format(tw)
    assert fast.shape == (S, m, 2, n)
    for i in range(m):
        for e in range(n):
            r = (e >> i) & 1
            pair = ((e >> (i + 1)) << i) | (e & ((1 << i) - 1))
            assert np.array_equal(fast[:, i, 0, e], tw[:, i, pair, r, r])
            assert np.array_equal(fast[:, i, 1, e], tw[:, i, pair, r, 1 - r])
    assert np.array_equal(lo.twiddle_fast_to_normal_format(fast), tw)
    x = rng.standard_normal((3, S, n))
    for inc in (True, False):
        f = fast if inc else fast[:, ::-1]
        assert np.allclose(lo.butterfly_mult_untied_fast(f, x, inc), lo.butterfly_mult_untied(tw, x, inc))


def _numeric_grad(fn, param, g, eps=1e-6):
    """Central differences of L = Re(sum(conj(g) * fn(param))) in every real coordinate."""
    out = np.zeros(param.shape, dtype=param.dtype)
    flat = param.reshape(-1)
    res = out.reshape(-1)
    for k in range(flat.size):
        for unit in ((1.0, 1j) if np.iscomplexobj(param) else (1.0,)):
            old = flat[k]
            flat[k] = old + eps * unit
            up = np.real(np.sum(np.conj(g) * fn(param)))
            flat[k] = old - eps * unit
            dn = np.real(np.sum(np.conj(g) * fn(param)))
            flat[k] = old
            res[k] += unit * (up - dn) / (2 * eps)
    return out


def test_legacy_gradients_against_central_differences():
    rng = np.random.default_rng(15)
    S, m, B = 2, 3, 3
    n = 1 << m
    for cplx in (False, True):
        x = _rand(rng, (B, S, n), cplx)
        g = _rand(rng, (B, S, n), cplx)
        for inc in (True, False):
            tied = _rand(rng, (S, n - 1, 2, 2), cplx)
            y, d_tw, d_x = lo.butterfly_mult(tied, x, inc, g)
            assert np.allclose(d_tw, _numeric_grad(lambda p: lo.butterfly_mult(p, x, inc), tied, g), atol=1e-6)
            assert np.allclose(d_x, _numeric_grad(lambda p: lo.butterfly_mult(tied, p, inc), x.copy(), g), atol=1e-6)
            untied = _rand(rng, (S, m, n // 2, 2, 2), cplx)
            y, d_tw, d_x = lo.butterfly_mult_untied(untied, x, inc, g)
            assert np.allclose(d_tw, _numeric_grad(lambda p: lo.butterfly_mult_untied(p, x, inc), untied, g), atol=1e-6)
            assert np.allclose(d_x, _numeric_grad(lambda p: lo.butterfly_mult_untied(untied, p, inc), x.copy(), g), atol=1e-6)
    x, g = rng.standard_normal((B, S, n)), rng.standard_normal((B, S, n))
    for inc in (True, False):
        th = rng.uniform(0, 6, (S, n - 1))
        _, d_th, d_x = lo.butterfly_ortho_mult_tied(th, x, inc, g)
        assert np.allclose(d_th, _numeric_grad(lambda p: lo.butterfly_ortho_mult_tied(p, x, inc), th, g), atol=1e-6)
        th = rng.uniform(0, 6, (S, m, n // 2))
        _, d_th, d_x = lo.butterfly_ortho_mult_untied(th, x, inc, g)
        assert np.allclose(d_th, _numeric_grad(lambda p: lo.butterfly_ortho_mult_untied(p, x, inc), th, g), atol=1e-6)
        assert np.allclose(d_x, _numeric_grad(lambda p: lo.butterfly_ortho_mult_untied(th, p, inc), x.copy(), g), atol=1e-6)
        fast = rng.standard_normal((S, m, 2, n))
        _, d_f, d_x = lo.butterfly_mult_untied_fast(fast, x, inc, g)
        assert np.allclose(d_f, _numeric_grad(lambda p: lo.butterfly_mult_untied_fast(p, x, inc), fast, g), atol=1e-6)
    tw = rng.standard_normal((S, 2 * 2 * m, n // 2, 2, 2))
    _, d_tw, d_x = lo.bbt_mult_untied(tw, x, g)
    assert np.allclose(d_tw, _numeric_grad(lambda p: lo.bbt_mult_untied(p, x), tw, g), atol=1e-6)
    assert np.allclose(d_x, _numeric_grad(lambda p: lo.bbt_mult_untied(tw, p), x.copy(), g), atol=1e-6)
    fast = rng.standard_normal((S, 2 * 2 * m, 2, n))
    _, d_f, d_x = lo.bbt_mult_untied_fast(fast, x, g)
    assert np.allclose(d_f, _numeric_grad(lambda p: lo.bbt_mult_untied_fast(p, x), fast, g), atol=1e-6)
    th = rng.uniform(0, 6, (S, 2 * 2 * m, n // 2))
    _, d_th, _ = lo.bbt_ortho_mult_untied(th, x, g)
    assert np.allclose(d_th, _numeric_grad(lambda p: lo.bbt_ortho_mult_untied(p, x), th, g), atol=1e-6)
    tht = rng.uniform(0, 6, (S, 4, n - 1))
    _, d_th, d_x = lo.bbt_ortho_mult_tied(tht, x, g)
    assert np.allclose(d_th, _numeric_grad(lambda p: lo.bbt_ortho_mult_tied(p, x), tht, g), atol=1e-6)
    diag = rng.standard_normal((S, 2, n))
    _, d_th, d_d, d_x = lo.odo_mult_untied(th, diag, x, g)
    assert np.allclose(d_th, _numeric_grad(lambda p: lo.odo_mult_untied(p, diag, x), th, g), atol=1e-6)
    assert np.allclose(d_d, _numeric_grad(lambda p: lo.odo_mult_untied(th, p, x), diag, g), atol=1e-6)
    assert np.allclose(d_x, _numeric_grad(lambda p: lo.odo_mult_untied(th, diag, p), x.copy(), g), atol=1e-6)
