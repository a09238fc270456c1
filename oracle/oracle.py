"""numpy front-end of the CPU oracle (TEST INFRASTRUCTURE ONLY).

Only tests, ``__graft_entry__.smoke`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this module; the product package never does.

The functions take and return numpy arrays and mirror the reference operator
semantics (csrc/butterfly.cpp:20-93): twiddle first, input zero-padded or trimmed to
``n``, output trimmed to ``output_size``, ``d_input`` the size of ``input``.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")
_lib = None

_SUFFIX = {np.dtype(np.float32): "f32", np.dtype(np.float64): "f64",
           np.dtype(np.complex64): "c64", np.dtype(np.complex128): "c128"}


def lib():
    global _lib
    if _lib is None:
        if not os.path.isfile(_SO):
            raise RuntimeError(f"{_SO} not built; run `python oracle/build.py`")
        _lib = ctypes.CDLL(_SO)
    return _lib


def _ptr(a):
    return ctypes.c_void_p(a.ctypes.data)


def _i64(v):
    return ctypes.c_int64(int(v))


def _prep(*arrays):
    dt = arrays[0].dtype
    if dt not in _SUFFIX:
        raise TypeError(f"unsupported dtype {dt}")
    out = []
    for a in arrays:
        if a.dtype != dt:
            raise TypeError("all operands must share one dtype")
        out.append(np.ascontiguousarray(a))
    return _SUFFIX[dt], out


def _check_twiddle(twiddle, S):
    if twiddle.ndim != 6:
        raise ValueError("twiddle must have dimension 6")
    S_, nb, L, half, a, b = twiddle.shape
    n = 1 << L
    if (S_, half, a, b) != (S, n // 2, 2, 2):
        raise ValueError("twiddle must have shape (nstacks, nblocks, log_n, n / 2, 2, 2)")
    return nb, L, n


def butterfly_fw(twiddle, input, increasing_stride=True, output_size=None):
    sfx, (twiddle, input) = _prep(twiddle, input)
    B, S, I = input.shape
    nb, L, n = _check_twiddle(twiddle, S)
    O = n if output_size is None else output_size
    if O > n:
        raise ValueError("output_size must be <= n")
    out = np.empty((B, S, n), dtype=input.dtype)
    fn = getattr(lib(), f"oracle_butterfly_fw_{sfx}")
    rc = fn(_ptr(twiddle), _ptr(input), _ptr(out), _i64(B), _i64(S), _i64(nb), _i64(L),
            _i64(I), ctypes.c_int(bool(increasing_stride)))
    assert rc == 0
    return out[:, :, :O]


def butterfly_bw(twiddle, input, grad, increasing_stride=True):
    sfx, (twiddle, input, grad) = _prep(twiddle, input, grad)
    B, S, I = input.shape
    nb, L, n = _check_twiddle(twiddle, S)
    O = grad.shape[2]
    if grad.shape != (B, S, O):
        raise ValueError("grad must have shape (batch_size, nstacks, output_size)")
    W = max(I, n)
    d_twiddle = np.empty_like(twiddle)
    d_input = np.empty((B, S, W), dtype=input.dtype)
    scratch = np.empty((max(nb * L, 1), B, S, n), dtype=input.dtype)
    fn = getattr(lib(), f"oracle_butterfly_bw_{sfx}")
    rc = fn(_ptr(twiddle), _ptr(input), _ptr(grad), _ptr(d_twiddle), _ptr(d_input),
            _ptr(scratch), _i64(B), _i64(S), _i64(nb), _i64(L), _i64(I), _i64(O),
            ctypes.c_int(bool(increasing_stride)))
    assert rc == 0
    return d_twiddle, d_input[:, :, :I]


def _check_base4(twiddle4, twiddle2, S):
    nb = twiddle4.shape[1]
    L = twiddle4.shape[2] * 2 + twiddle2.shape[2]
    n = 1 << L
    if L // 2 > 0 and twiddle4.shape != (S, nb, L // 2, n // 4, 4, 4):
        raise ValueError("twiddle4 must have shape (nstacks, nblocks, log_n / 2, n / 4, 4, 4)")
    if L % 2 == 1 and twiddle2.shape != (S, nb, 1, n // 2, 2, 2):
        raise ValueError("twiddle2 must have shape (nstacks, nblocks, 1, n / 2, 2, 2)")
    return nb, L, n


def butterfly_base4_fw(twiddle4, twiddle2, input, increasing_stride=True, output_size=None):
    sfx, (twiddle4, twiddle2, input) = _prep(twiddle4, twiddle2, input)
    B, S, I = input.shape
    nb, L, n = _check_base4(twiddle4, twiddle2, S)
    O = n if output_size is None else output_size
    if O > n:
        raise ValueError("output_size must be <= n")
    out = np.empty((B, S, n), dtype=input.dtype)
    fn = getattr(lib(), f"oracle_butterfly_base4_fw_{sfx}")
    rc = fn(_ptr(twiddle4), _ptr(twiddle2), _ptr(input), _ptr(out), _i64(B), _i64(S),
            _i64(nb), _i64(L), _i64(I), ctypes.c_int(bool(increasing_stride)))
    assert rc == 0
    return out[:, :, :O]


def butterfly_base4_bw(twiddle4, twiddle2, input, grad, increasing_stride=True):
    sfx, (twiddle4, twiddle2, input, grad) = _prep(twiddle4, twiddle2, input, grad)
    B, S, I = input.shape
    nb, L, n = _check_base4(twiddle4, twiddle2, S)
    O = grad.shape[2]
    W = max(I, n)
    per = L // 2 + L % 2
    d4 = np.empty_like(twiddle4)
    d2 = np.empty_like(twiddle2)
    d_input = np.empty((B, S, W), dtype=input.dtype)
    scratch = np.empty((max(nb * per, 1), B, S, n), dtype=input.dtype)
    fn = getattr(lib(), f"oracle_butterfly_base4_bw_{sfx}")
    rc = fn(_ptr(twiddle4), _ptr(twiddle2), _ptr(input), _ptr(grad), _ptr(d4), _ptr(d2),
            _ptr(d_input), _ptr(scratch), _i64(B), _i64(S), _i64(nb), _i64(L), _i64(I),
            _i64(O), ctypes.c_int(bool(increasing_stride)))
    assert rc == 0
    return d4, d2, d_input[:, :, :I]


def twiddle_base2_to_base4(twiddle, increasing_stride=True):
    """Fuse stage pairs (2 idx, 2 idx + 1) of every block into one 4x4 factor per quad.

    Functional restatement of torch_butterfly/multiply_base4.py:44-71: for quad q of the
    radix-4 stage with stride st, T4 = (stage 2 idx + 1) o (stage 2 idx) restricted to the
    elements {pos + c st}.  With increasing stride the earlier stage pairs (c, c^1) at
    stride st and the later (c, c^2) at 2 st; with decreasing stride the other way round.
    """
    S, nb, L = twiddle.shape[:3]
    n = 1 << L
    L4 = L // 2
    tw2 = twiddle[:, :, -1:].copy() if L % 2 == 1 else np.empty((S, nb, 0, n // 2, 2, 2), twiddle.dtype)
    tw4 = np.zeros((S, nb, L4, n // 4, 4, 4), dtype=twiddle.dtype)
    for block in range(nb):
        cur_inc = bool(increasing_stride) != bool(block % 2)
        for idx in range(L4):
            l2 = 2 * idx if cur_inc else L - 2 - 2 * idx
            st = 1 << l2
            # strides of the two fused base-2 stages, in execution order
            s_first, s_second = (st, 2 * st) if cur_inc else (2 * st, st)
            for q in range(n // 4):
                low = q % st
                pos = 4 * (q - low) + low
                elems = [pos + c * st for c in range(4)]
                mats = []
                for stage, sstride in ((2 * idx, s_first), (2 * idx + 1, s_second)):
                    M = np.zeros((S, 4, 4), dtype=twiddle.dtype)
                    for c, e in enumerate(elems):
                        if e & sstride:
                            continue
                        lowb = e % sstride
                        i = (e - lowb) // 2 + lowb
                        c1 = elems.index(e + sstride)
                        t = twiddle[:, block, stage, i]
                        M[:, c, c] = t[:, 0, 0]
                        M[:, c, c1] = t[:, 0, 1]
                        M[:, c1, c] = t[:, 1, 0]
                        M[:, c1, c1] = t[:, 1, 1]
                    mats.append(M)
                tw4[:, block, idx, q] = np.einsum("sij,sjk->sik", mats[1], mats[0])
    return tw4, tw2
