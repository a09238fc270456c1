"""Write ``tests/golden/butterfly_ref_cases.npz``: seeded operands plus the outputs the
compiled reference C++ (``oracle/_ref``, built by ``oracle/build.py`` from
``/root/reference/csrc``) returns for them.  Needs the reference tree; the committed
archive is what travels.

    python oracle/build.py && python tests/golden/make_golden.py
"""
import os
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OUT = os.path.join(HERE, "butterfly_ref_cases.npz")

DTYPES = [np.float32, np.float64, np.complex64, np.complex128]


def randn(rng, shape, dtype):
    dtype = np.dtype(dtype)
    if dtype.kind == "c":
        z = (rng.standard_normal(shape) + 1j * rng.standard_normal(shape)) / np.sqrt(2)
        return z.astype(dtype)
    return rng.standard_normal(shape).astype(dtype)


def cases():
    """(dtype, B, S, L, nb, input_size, output_size or -1, increasing_stride)."""
    out = []
    for dt in DTYPES:
        for inc in (1, 0):
            for nb in (1, 2, 3):
                out.append((dt, 3, 2, 4, nb, 16, -1, inc))
            # padded / trimmed input, sliced output (tests/test_multiply.py:61-90 of the reference)
            out.append((dt, 2, 2, 5, 3, 15, -1, inc))
            out.append((dt, 2, 2, 5, 3, 28, 14, inc))
            out.append((dt, 2, 2, 5, 2, 71, 27, inc))
    # smallest sizes
    out.append((np.float32, 4, 1, 1, 1, 2, -1, 1))
    out.append((np.float32, 4, 1, 1, 2, 2, -1, 0))
    out.append((np.complex64, 2, 3, 2, 2, 4, -1, 1))
    # a longer vector
    out.append((np.float32, 2, 1, 8, 2, 256, -1, 0))
    out.append((np.complex64, 2, 1, 7, 1, 128, -1, 1))
    return out


def main():
    rng = np.random.default_rng(20240607)
    blob = {}
    for i, (dt, B, S, L, nb, I, O, inc) in enumerate(cases()):
        n = 1 << L
        blob[f"c{i}_twiddle"] = (randn(rng, (S, nb, L, n // 2, 2, 2), dt) / np.sqrt(2)).astype(dt)
        blob[f"c{i}_input"] = randn(rng, (B, S, I), dt)
        blob[f"c{i}_grad"] = randn(rng, (B, S, n if O < 0 else O), dt)
        blob[f"c{i}_meta"] = np.array([inc, O], dtype=np.int64)
    with tempfile.TemporaryDirectory() as tmp:
        fin, fout = os.path.join(tmp, "in.npz"), os.path.join(tmp, "out.npz")
        np.savez(fin, **blob)
        subprocess.check_call([sys.executable, os.path.join(ROOT, "oracle", "ref_runner.py"),
                               "run", fin, fout])
        res = np.load(fout)
        for k in res.files:
            blob[k] = res[k]
    np.savez_compressed(OUT, **blob)
    print(f"wrote {OUT}: {len(cases())} cases, {os.path.getsize(OUT) / 1024:.0f} KiB")


if __name__ == "__main__":
    main()
