"""CPU restatement of the legacy ``butterfly`` package's multiply functions (TEST
INFRASTRUCTURE ONLY: only tests may import this module; the product package never does).

The legacy package (reference: butterfly/butterfly_multiply.py, butterfly/utils.py) is not
importable in this build's environment (it needs apex and its own compiled extensions), so
its algorithm is restated here in numpy from the plain-PyTorch definitions it carries, and
from the relations its own tests state for the functions that only exist as CUDA code
(tests_old/test_butterfly_multiply.py:320-368, 427-474, 556-600).

Every function is a sequence of two kinds of steps, applied literally one after the other --
``factor`` (one butterfly factor of a given stride) and ``diag`` (an elementwise scale) --
followed, for the gradients, by the adjoint steps in reverse order and the chain rule through
the parameterisation (tied weights, rotation angles).  Nothing is folded or reordered, so this
file shares no index arithmetic with the adapter it checks.

Complex data: numpy complex arrays stand for the legacy (..., 2) real pairs; gradients follow
the convention d_param = sum g * conj(x), which is what autograd gives for the real pairs.

Pinned by tests/test_oracle.py::test_legacy_* : each factor against a dense matrix built
entry by entry from the definition, the tied product against numpy's FFT (radix-2 decimation
in time, a non-symmetric 2x2 per pair), the rotation's sign on a 2-point case, the fast
format against its element formula, gradients against central differences in float64.
"""
import numpy as np


# ---- the two steps and their adjoints ---------------------------------------------------------

def factor_apply(T, log_stride, x):
    """One butterfly factor: T (S, n/2, 2, 2), pair i = h * stride + l couples the elements
    h * 2 stride + l and h * 2 stride + stride + l; out_r = sum_c T[i][r][c] in_c
    (butterfly_multiply.py:147-150: view (n / 2 stride, stride, 2, 2), product with the input
    viewed as (n / 2 stride, 1, 2, stride), sum over the input's pair axis)."""
    B, S, n = x.shape
    st = 1 << log_stride
    t = T.reshape(S, n // (2 * st), st, 2, 2)
    xv = x.reshape(B, S, n // (2 * st), 2, st)
    return np.einsum("shlrc,bshcl->bshrl", t, xv).reshape(B, S, n)


def factor_adjoint(T, log_stride, x, g):
    """(d_T, d_x) of factor_apply for the output gradient g."""
    B, S, n = x.shape
    st = 1 << log_stride
    t = T.reshape(S, n // (2 * st), st, 2, 2)
    xv = x.reshape(B, S, n // (2 * st), 2, st)
    gv = g.reshape(B, S, n // (2 * st), 2, st)
    d_t = np.einsum("bshrl,bshcl->shlrc", gv, np.conj(xv)).reshape(T.shape)
    d_x = np.einsum("shlrc,bshrl->bshcl", np.conj(t), gv).reshape(B, S, n)
    return d_t, d_x


def _run(steps, x, g=None):
    """steps: list of ("factor", T, log_stride) / ("diag", d (S, n)).  Returns the output, and
    with g also the per-step parameter gradients and d_x."""
    inputs = []
    for step in steps:
        inputs.append(x)
        x = factor_apply(step[1], step[2], x) if step[0] == "factor" else x * step[1][None]
    if g is None:
        return x
    grads = [None] * len(steps)
    for k in range(len(steps) - 1, -1, -1):
        step = steps[k]
        if step[0] == "factor":
            grads[k], g = factor_adjoint(step[1], step[2], inputs[k], g)
        else:
            grads[k] = np.einsum("bsn,bsn->sn", g, np.conj(inputs[k]))
            g = g * np.conj(step[1])[None]
    return x, grads, g


# ---- parameterisations ----------------------------------------------------------------------------

def tied_expand(tied, log_stride, n):
    """Factor of a tied twiddle (S, n - 1, 2, 2): entries stride - 1 .. 2 stride - 2, shared by
    all n / (2 stride) groups (butterfly_multiply.py:64-66)."""
    st = 1 << log_stride
    t = tied[:, st - 1:2 * st - 1]                                   # (S, stride, 2, 2)
    return np.broadcast_to(t[:, None], (t.shape[0], n // (2 * st), st, 2, 2)).reshape(t.shape[0], n // 2, 2, 2)


def tied_collect(d_T, log_stride, n):
    """Adjoint of tied_expand: sum over the groups.  Returns (S, stride, 2, 2)."""
    st = 1 << log_stride
    return d_T.reshape(d_T.shape[0], n // (2 * st), st, 2, 2).sum(axis=1)


def rotation(theta):
    """[[cos, -sin], [sin, cos]] per angle (butterfly_multiply.py:265-269, 315-319)."""
    c, s = np.cos(theta), np.sin(theta)
    return np.stack((np.stack((c, -s), -1), np.stack((s, c), -1)), -2)


def rotation_adjoint(theta, d_T):
    """d_theta from the gradient of the four entries."""
    c, s = np.cos(theta), np.sin(theta)
    return (-s * d_T[..., 0, 0] - c * d_T[..., 0, 1] + c * d_T[..., 1, 0] - s * d_T[..., 1, 1])


def _order(m, increasing_stride):
    return list(range(m)) if increasing_stride else list(range(m - 1, -1, -1))


# ---- the legacy functions ---------------------------------------------------------------------------

def butterfly_mult(twiddle, x, increasing_stride=True, g=None):
    """Tied weights, twiddle (S, n - 1, 2, 2) (butterfly_multiply.py:43-79).
    With g: (y, d_twiddle, d_x)."""
    n = x.shape[2]
    m = n.bit_length() - 1
    order = _order(m, increasing_stride)
    steps = [("factor", tied_expand(twiddle, ls, n), ls) for ls in order]
    if g is None:
        return _run(steps, x)
    y, grads, d_x = _run(steps, x, g)
    d_tw = np.zeros_like(twiddle)
    for ls, d_T in zip(order, grads):
        st = 1 << ls
        d_tw[:, st - 1:2 * st - 1] += tied_collect(d_T, ls, n)
    return y, d_tw, d_x


def butterfly_mult_untied(twiddle, x, increasing_stride=True, g=None):
    """twiddle (S, log n, n / 2, 2, 2), twiddle[:, log_stride] always belongs to that stride
    whatever the order (butterfly_multiply.py:126-162)."""
    n = x.shape[2]
    m = n.bit_length() - 1
    order = _order(m, increasing_stride)
    steps = [("factor", twiddle[:, ls], ls) for ls in order]
    if g is None:
        return _run(steps, x)
    y, grads, d_x = _run(steps, x, g)
    d_tw = np.zeros_like(twiddle)
    for ls, d_T in zip(order, grads):
        d_tw[:, ls] = d_T
    return y, d_tw, d_x


def butterfly_ortho_mult_tied(theta, x, increasing_stride, g=None):
    """theta (S, n - 1) (butterfly_multiply.py:265-269)."""
    if g is None:
        return butterfly_mult(rotation(theta), x, increasing_stride)
    y, d_tw, d_x = butterfly_mult(rotation(theta), x, increasing_stride, g)
    return y, rotation_adjoint(theta, d_tw), d_x


def butterfly_ortho_mult_untied(theta, x, increasing_stride, g=None):
    """theta (S, log n, n / 2) (butterfly_multiply.py:315-319)."""
    if g is None:
        return butterfly_mult_untied(rotation(theta), x, increasing_stride)
    y, d_tw, d_x = butterfly_mult_untied(rotation(theta), x, increasing_stride, g)
    return y, rotation_adjoint(theta, d_tw), d_x


def _bbt_steps(twiddle, n):
    """Steps of bbt_mult_untied_torch (butterfly_multiply.py:377-386): per block of 2 log n
    factors, the first log n flipped and applied with decreasing stride, the rest with
    increasing stride.  Returns (steps, index of the twiddle slice each step came from)."""
    m = n.bit_length() - 1
    nblocks = twiddle.shape[1] // (2 * m)
    steps, src = [], []
    for b in range(nblocks):
        base = b * 2 * m
        first = twiddle[:, base:base + m][:, ::-1]          # .flip(1): first[log_stride]
        for ls in _order(m, False):
            steps.append(("factor", first[:, ls], ls))
            src.append(base + (m - 1 - ls))
        second = twiddle[:, base + m:base + 2 * m]
        for ls in _order(m, True):
            steps.append(("factor", second[:, ls], ls))
            src.append(base + m + ls)
    return steps, src


def bbt_mult_untied(twiddle, x, g=None):
    """twiddle (S, nblocks * 2 log n, n / 2, 2, 2)."""
    steps, src = _bbt_steps(twiddle, x.shape[2])
    if g is None:
        return _run(steps, x)
    y, grads, d_x = _run(steps, x, g)
    d_tw = np.zeros_like(twiddle)
    for k, d_T in zip(src, grads):
        d_tw[:, k] = d_T
    return y, d_tw, d_x


def bbt_ortho_mult_untied(theta, x, g=None):
    """theta (S, nblocks * 2 log n, n / 2) (butterfly_multiply.py:444-449)."""
    if g is None:
        return bbt_mult_untied(rotation(theta), x)
    y, d_tw, d_x = bbt_mult_untied(rotation(theta), x, g)
    return y, rotation_adjoint(theta, d_tw), d_x


def bbt_ortho_mult_tied(theta, x, g=None):
    """theta (S, nblocks * 2, n - 1): per block, slice 0 with decreasing and slice 1 with
    increasing stride (butterfly_multiply.py:389-398)."""
    n = x.shape[2]
    m = n.bit_length() - 1
    steps, src = [], []
    for k in range(theta.shape[1]):
        T = rotation(theta[:, k])
        for ls in _order(m, k % 2 == 1):
            steps.append(("factor", tied_expand(T, ls, n), ls))
            src.append((k, ls))
    if g is None:
        return _run(steps, x)
    y, grads, d_x = _run(steps, x, g)
    d_T = np.zeros(theta.shape + (2, 2), dtype=x.dtype)
    for (k, ls), d in zip(src, grads):
        st = 1 << ls
        d_T[:, k, st - 1:2 * st - 1] += tied_collect(d, ls, n)
    return y, rotation_adjoint(theta, d_T), d_x


def odo_mult_untied(theta, diag, x, g=None):
    """theta (S, nblocks * 2 log n, n / 2), diag (S, nblocks, n): per block an orthogonal
    butterfly with decreasing stride from the flipped first log n slices, the diagonal, an
    orthogonal butterfly with increasing stride from the rest
    (tests_old/test_butterfly_multiply.py:575-579 states this for the CUDA-only kernel).
    With g: (y, d_theta, d_diag, d_x)."""
    n = x.shape[2]
    m = n.bit_length() - 1
    nblocks = theta.shape[1] // (2 * m)
    T = rotation(theta)
    steps, src = [], []
    for b in range(nblocks):
        base = b * 2 * m
        first = T[:, base:base + m][:, ::-1]
        for ls in _order(m, False):
            steps.append(("factor", first[:, ls], ls))
            src.append(base + (m - 1 - ls))
        steps.append(("diag", diag[:, b]))
        src.append(("diag", b))
        second = T[:, base + m:base + 2 * m]
        for ls in _order(m, True):
            steps.append(("factor", second[:, ls], ls))
            src.append(base + m + ls)
    if g is None:
        return _run(steps, x)
    y, grads, d_x = _run(steps, x, g)
    d_T = np.zeros_like(T)
    d_diag = np.zeros_like(diag)
    for k, d in zip(src, grads):
        if isinstance(k, tuple):
            d_diag[:, k[1]] = d
        else:
            d_T[:, k] = d
    return y, rotation_adjoint(theta, d_T), d_diag, d_x


# ---- fast format ------------------------------------------------------------------------------------

def twiddle_normal_to_fast_format(twiddle):
    """(S, log n, n / 2, 2, 2) -> (S, log n, 2, n), operation by operation as in
    butterfly/utils.py:24-45: swap the second row's two entries, then per stride regroup
    (groups, stride, row, col) as (groups, row, stride, col) and move col in front."""
    tw = twiddle.copy()
    S, m, half = tw.shape[:3]
    n = 2 * half
    tw[:, :, :, 1] = tw[:, :, :, 1][..., [1, 0]]
    out = []
    for i in range(m):
        st = 1 << i
        t = tw[:, i].reshape(S, n // 2 // st, st, 2, 2).transpose(0, 1, 3, 2, 4)
        out.append(t.reshape(S, n, 2).transpose(0, 2, 1))
    return np.stack(out, axis=1)


def twiddle_fast_to_normal_format(fast):
    """Inverse of the above, written from its element formula: position e of stride-2^i's
    slice belongs to pair i(e) (e with bit i removed) and row r = bit i of e; plane 0 holds
    T[r][r], plane 1 holds T[r][1 - r]."""
    S, m, _, n = fast.shape
    tw = np.zeros((S, m, n // 2, 2, 2), dtype=fast.dtype)
    for i in range(m):
        st = 1 << i
        for e in range(n):
            r = (e >> i) & 1
            pair = ((e >> (i + 1)) << i) | (e & (st - 1))
            tw[:, i, pair, r, r] = fast[:, i, 0, e]
            tw[:, i, pair, r, 1 - r] = fast[:, i, 1, e]
    return tw


def butterfly_mult_untied_fast(twiddle_fast, x, increasing_stride=True, g=None):
    """The fast-format entry: twiddle_fast is the converted twiddle, flipped along the stride
    axis for decreasing stride; gradients come back in the same format
    (tests_old/test_butterfly_multiply.py:335-366)."""
    fast = twiddle_fast if increasing_stride else twiddle_fast[:, ::-1]
    tw = twiddle_fast_to_normal_format(fast)
    if g is None:
        return butterfly_mult_untied(tw, x, increasing_stride)
    y, d_tw, d_x = butterfly_mult_untied(tw, x, increasing_stride, g)
    d_fast = twiddle_normal_to_fast_format(d_tw)
    return y, (d_fast if increasing_stride else d_fast[:, ::-1]), d_x


def bbt_mult_untied_fast(twiddle_fast, x, g=None):
    """Fast-format B B^T product: per slice of log n factors the converted twiddle, even
    slices flipped; in normal format even slices run with decreasing and odd slices with
    increasing stride, none of them flipped (tests_old/test_butterfly_multiply.py:441-470)."""
    n = x.shape[2]
    m = n.bit_length() - 1
    nchunks = twiddle_fast.shape[1] // m
    tws = []
    for k in range(nchunks):
        chunk = twiddle_fast[:, k * m:(k + 1) * m]
        tws.append(twiddle_fast_to_normal_format(chunk[:, ::-1] if k % 2 == 0 else chunk))
    steps, src = [], []
    for k in range(nchunks):
        for ls in _order(m, k % 2 == 1):
            steps.append(("factor", tws[k][:, ls], ls))
            src.append((k, ls))
    if g is None:
        return _run(steps, x)
    y, grads, d_x = _run(steps, x, g)
    d_tws = [np.zeros_like(t) for t in tws]
    for (k, ls), d in zip(src, grads):
        d_tws[k][:, ls] = d
    d_fast = []
    for k in range(nchunks):
        f = twiddle_normal_to_fast_format(d_tws[k])
        d_fast.append(f[:, ::-1] if k % 2 == 0 else f)
    return y, np.concatenate(d_fast, axis=1), d_x
