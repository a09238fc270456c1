"""ctypes binding of the C ABI in ``include/butterfly_hip.h`` (``libbutterfly_hip.so``).

Used by the parity tests and the benchmark to call the library below the operator shim,
with raw device pointers taken from torch tensors.
"""
import ctypes
import os

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libbutterfly_hip.so")

BF_F32, BF_C64 = 0, 1
BF_ERR_INVALID, BF_ERR_UNSUPPORTED, BF_ERR_HIP, BF_ERR_WORKSPACE = -1, -2, -3, -4

SYMBOLS = [
    "bf_version", "bf_hip_version", "bf_last_error",
    "bf_butterfly_multiply_fw", "bf_butterfly_multiply_fw_workspace_bytes",
    "bf_butterfly_multiply_bw_workspace_bytes", "bf_butterfly_multiply_bw",
    "bf_butterfly_multiply_bias_fw", "bf_butterfly_bias_grad", "bf_butterfly_bias_grad_workspace_bytes",
    "bf_butterfly_multiply_bias_bw", "bf_butterfly_multiply_bias_bw_workspace_bytes",
    "bf_butterfly_multiply_perm_fw", "bf_butterfly_multiply_perm_bw", "bf_describe_plan",
    "bf_butterfly_scale_twiddle", "bf_butterfly_scale_twiddle_bw",
    "bf_butterfly_multiply_base4_fw", "bf_butterfly_multiply_base4_fw_workspace_bytes",
    "bf_butterfly_multiply_base4_bw_workspace_bytes",
    "bf_butterfly_multiply_base4_bw",
    "bf_butterfly_multiply_bw_noalloc",
    "bf_butterfly_multiply_saved_bytes", "bf_butterfly_multiply_fw_saving",
    "bf_butterfly_multiply_bw_saved_workspace_bytes", "bf_butterfly_multiply_bw_saved",
    "bf_butterfly_multiply_base4_saved_bytes", "bf_butterfly_multiply_base4_fw_saving",
    "bf_butterfly_multiply_base4_bw_saved_workspace_bytes", "bf_butterfly_multiply_base4_bw_saved",
]

NOALLOC_SCRATCH_BYTES = 48 << 20


class Problem(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int32),
        ("increasing_stride", ctypes.c_int32),
        ("batch", ctypes.c_int64),
        ("nstacks", ctypes.c_int64),
        ("log_n", ctypes.c_int64),
        ("nblocks", ctypes.c_int64),
        ("input_size", ctypes.c_int64),
        ("output_size", ctypes.c_int64),
        ("input_stride", ctypes.c_int64 * 3),
        ("output_stride", ctypes.c_int64 * 3),
        ("d_input_stride", ctypes.c_int64 * 3),
    ]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.isfile(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: run `python -m butterfly_amd.build`")
        L = ctypes.CDLL(LIB_PATH)
        vp, sz = ctypes.c_void_p, ctypes.c_size_t
        pp = ctypes.POINTER(Problem)
        L.bf_version.restype = ctypes.c_int
        L.bf_hip_version.restype = ctypes.c_int
        L.bf_last_error.restype = ctypes.c_char_p
        L.bf_butterfly_multiply_fw.argtypes = [pp, vp, vp, vp, vp, sz, vp]
        L.bf_butterfly_multiply_fw_workspace_bytes.argtypes = [pp]
        L.bf_butterfly_multiply_fw_workspace_bytes.restype = sz
        L.bf_butterfly_multiply_bw_workspace_bytes.argtypes = [pp]
        L.bf_butterfly_multiply_bw_workspace_bytes.restype = sz
        L.bf_butterfly_multiply_bw.argtypes = [pp, vp, vp, vp, vp, vp, vp, sz, vp]
        L.bf_butterfly_multiply_bias_fw.argtypes = [pp, vp, vp, vp, vp, vp, sz, vp]
        L.bf_butterfly_bias_grad.argtypes = [pp, vp, vp, vp, sz, vp]
        L.bf_butterfly_bias_grad_workspace_bytes.argtypes = [pp]
        L.bf_butterfly_bias_grad_workspace_bytes.restype = sz
        L.bf_butterfly_multiply_bias_bw.argtypes = [pp, vp, vp, vp, vp, vp, vp, vp, sz, vp]
        L.bf_butterfly_multiply_bias_bw_workspace_bytes.argtypes = [pp]
        L.bf_butterfly_multiply_bias_bw_workspace_bytes.restype = sz
        L.bf_butterfly_multiply_perm_fw.argtypes = [pp, vp, vp, vp, vp, vp, vp, vp, sz, vp]
        L.bf_butterfly_multiply_perm_bw.argtypes = [pp, vp, vp, vp, vp, vp, vp, vp, vp, vp, sz, vp]
        L.bf_describe_plan.argtypes = [pp, ctypes.c_int, ctypes.c_char_p, sz]
        i32, i64 = ctypes.c_int, ctypes.c_int64
        L.bf_butterfly_scale_twiddle.argtypes = [i32, i64, i64, i64, i32, vp, vp, i64, vp, i64, vp, vp]
        L.bf_butterfly_scale_twiddle_bw.argtypes = [i32, i64, i64, i64, i32, vp, vp, i64, vp, i64, vp, vp, vp, vp, vp]
        L.bf_butterfly_multiply_base4_fw.argtypes = [pp, vp, vp, vp, vp, vp, sz, vp]
        L.bf_butterfly_multiply_base4_fw_workspace_bytes.argtypes = [pp]
        L.bf_butterfly_multiply_base4_fw_workspace_bytes.restype = sz
        L.bf_butterfly_multiply_base4_bw_workspace_bytes.argtypes = [pp]
        L.bf_butterfly_multiply_base4_bw_workspace_bytes.restype = sz
        L.bf_butterfly_multiply_base4_bw.argtypes = [pp, vp, vp, vp, vp, vp, vp, vp, vp, sz, vp]
        L.bf_butterfly_multiply_bw_noalloc.argtypes = [pp, vp, vp, vp, vp, vp, vp]
        L.bf_butterfly_multiply_saved_bytes.argtypes = [pp]
        L.bf_butterfly_multiply_saved_bytes.restype = sz
        L.bf_butterfly_multiply_fw_saving.argtypes = [pp, vp, vp, vp, vp, vp, vp, vp, sz, vp]
        L.bf_butterfly_multiply_bw_saved_workspace_bytes.argtypes = [pp, ctypes.c_int]
        L.bf_butterfly_multiply_bw_saved_workspace_bytes.restype = sz
        L.bf_butterfly_multiply_bw_saved.argtypes = [pp, vp, vp, vp, vp, sz, vp, vp, vp, vp, vp, vp, sz, vp]
        L.bf_butterfly_multiply_base4_saved_bytes.argtypes = [pp]
        L.bf_butterfly_multiply_base4_saved_bytes.restype = sz
        L.bf_butterfly_multiply_base4_fw_saving.argtypes = [pp, vp, vp, vp, vp, vp, sz, vp]
        L.bf_butterfly_multiply_base4_bw_saved_workspace_bytes.argtypes = [pp]
        L.bf_butterfly_multiply_base4_bw_saved_workspace_bytes.restype = sz
        L.bf_butterfly_multiply_base4_bw_saved.argtypes = [pp, vp, vp, vp, vp, vp, sz, vp, vp, vp, vp, sz, vp]
        _lib = L
    return _lib


class ButterflyError(RuntimeError):
    def __init__(self, code):
        self.code = code
        super().__init__(f"libbutterfly_hip error {code}: {lib().bf_last_error().decode()}")


def _check(rc):
    if rc != 0:
        raise ButterflyError(rc)


SIZE_INVALID = ctypes.c_size_t(-1).value   # BF_SIZE_INVALID: the size queries' answer for a refused problem


def _size(nbytes):
    if nbytes == SIZE_INVALID:
        raise ButterflyError(BF_ERR_INVALID)
    return nbytes


def _dtype_code(t):
    if t.dtype == torch.float32:
        return BF_F32
    if t.dtype == torch.complex64:
        return BF_C64
    raise TypeError(f"unsupported dtype {t.dtype}")


def _strides(t):
    return (ctypes.c_int64 * 3)(*[t.stride(i) if t.size(i) > 1 else 0 for i in range(3)])


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None and t.numel() > 0 else ctypes.c_void_p(0)


def make_problem(input, log_n, nblocks, increasing_stride, output_size):
    p = Problem()
    p.dtype = _dtype_code(input)
    p.increasing_stride = int(bool(increasing_stride))
    p.batch, p.nstacks, p.input_size = input.shape
    p.log_n, p.nblocks = log_n, nblocks
    p.output_size = output_size
    p.input_stride = _strides(input)
    return p


def multiply_fw(twiddle, input, increasing_stride, output_size=None):
    """Forward through the C ABI; twiddle must be dense.  Returns (B, S, output_size)."""
    assert twiddle.is_contiguous() and twiddle.is_cuda and input.is_cuda
    nb, log_n = twiddle.shape[1], twiddle.shape[2]
    n = 1 << log_n
    O = n if output_size is None else output_size
    p = make_problem(input, log_n, nb, increasing_stride, O)
    out = torch.empty(input.shape[0], input.shape[1], O, dtype=input.dtype, device=input.device)
    p.output_stride = _strides(out)
    nbytes = _size(lib().bf_butterfly_multiply_fw_workspace_bytes(ctypes.byref(p)))
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=input.device)
    _check(lib().bf_butterfly_multiply_fw(ctypes.byref(p), _ptr(twiddle), _ptr(input), _ptr(out), _ptr(ws), nbytes,
                                          _stream()))
    return out


def multiply_bias_fw(twiddle, input, bias, increasing_stride, output_size=None):
    """Forward with the bias (S, output_size) added by the library."""
    assert twiddle.is_contiguous() and twiddle.is_cuda and input.is_cuda
    nb, log_n = twiddle.shape[1], twiddle.shape[2]
    n = 1 << log_n
    O = n if output_size is None else output_size
    assert bias.is_contiguous() and tuple(bias.shape) == (input.shape[1], O) and bias.dtype == input.dtype
    p = make_problem(input, log_n, nb, increasing_stride, O)
    out = torch.empty(input.shape[0], input.shape[1], O, dtype=input.dtype, device=input.device)
    p.output_stride = _strides(out)
    nbytes = _size(lib().bf_butterfly_multiply_fw_workspace_bytes(ctypes.byref(p)))
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=input.device)
    _check(lib().bf_butterfly_multiply_bias_fw(ctypes.byref(p), _ptr(twiddle), _ptr(input), _ptr(bias), _ptr(out),
                                               _ptr(ws), nbytes, _stream()))
    return out


def bias_grad(grad):
    """Column sums of grad (B, S, O) over the batch, (S, O)."""
    assert grad.is_cuda and grad.dim() == 3
    p = Problem()
    p.dtype = _dtype_code(grad)
    p.batch, p.nstacks, p.output_size = grad.shape
    p.input_size = grad.shape[2]
    p.log_n = max(1, (int(grad.shape[2]) - 1).bit_length())
    p.nblocks = 1
    p.output_stride = _strides(grad)
    d_bias = torch.empty(grad.shape[1], grad.shape[2], dtype=grad.dtype, device=grad.device)
    nbytes = _size(lib().bf_butterfly_bias_grad_workspace_bytes(ctypes.byref(p)))
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=grad.device)
    _check(lib().bf_butterfly_bias_grad(ctypes.byref(p), _ptr(grad), _ptr(d_bias), _ptr(ws), nbytes, _stream()))
    return d_bias


def multiply_bias_bw(twiddle, input, grad, increasing_stride):
    """Backward that also returns d_bias (S, O).  Returns (d_twiddle, d_input, d_bias)."""
    assert twiddle.is_contiguous() and twiddle.is_cuda and input.is_cuda and grad.is_cuda
    nb, log_n = twiddle.shape[1], twiddle.shape[2]
    p = make_problem(input, log_n, nb, increasing_stride, grad.shape[2])
    p.output_stride = _strides(grad)
    d_twiddle = torch.empty_like(twiddle)
    d_input = torch.empty(input.shape, dtype=input.dtype, device=input.device)
    d_bias = torch.empty(grad.shape[1], grad.shape[2], dtype=grad.dtype, device=grad.device)
    p.d_input_stride = _strides(d_input)
    nbytes = _size(lib().bf_butterfly_multiply_bias_bw_workspace_bytes(ctypes.byref(p)))
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=input.device)
    _check(lib().bf_butterfly_multiply_bias_bw(ctypes.byref(p), _ptr(twiddle), _ptr(input), _ptr(grad),
                                               _ptr(d_twiddle), _ptr(d_input), _ptr(d_bias), _ptr(ws), nbytes,
                                               _stream()))
    return d_twiddle, d_input, d_bias


def describe_plan(dtype_code, batch, nstacks, log_n, nblocks, increasing_stride, backward):
    """The launch plan of a dense base-2 problem as a list of text lines (host only)."""
    n = 1 << log_n
    p = Problem()
    p.dtype, p.increasing_stride = dtype_code, int(increasing_stride)
    p.batch, p.nstacks, p.log_n, p.nblocks = batch, nstacks, log_n, nblocks
    p.input_size = p.output_size = n
    dense = (ctypes.c_int64 * 3)(nstacks * n, n, 1)
    p.input_stride = p.output_stride = p.d_input_stride = dense
    buf = ctypes.create_string_buffer(1 << 14)
    _check(lib().bf_describe_plan(ctypes.byref(p), int(backward), buf, len(buf)))
    return buf.value.decode().splitlines()


def _scale_args(twiddle, in_scale, out_scale):
    assert twiddle.is_cuda and twiddle.is_contiguous() and twiddle.dim() == 6
    for v in (in_scale, out_scale):
        assert v is None or (v.is_cuda and v.is_contiguous() and v.dim() == 1 and v.dtype == twiddle.dtype)
    return (_dtype_code(twiddle), twiddle.shape[0], twiddle.shape[1], twiddle.shape[2])


def scale_twiddle(twiddle, in_scale, out_scale, increasing_stride):
    """Factors of diag(out_scale) B diag(in_scale) (either scale may be None)."""
    head = _scale_args(twiddle, in_scale, out_scale)
    out = torch.empty_like(twiddle)
    _check(lib().bf_butterfly_scale_twiddle(
        *head, int(increasing_stride), _ptr(twiddle),
        None if in_scale is None else _ptr(in_scale), 0 if in_scale is None else in_scale.numel(),
        None if out_scale is None else _ptr(out_scale), 0 if out_scale is None else out_scale.numel(),
        _ptr(out), _stream()))
    return out


def scale_twiddle_bw(twiddle, in_scale, out_scale, increasing_stride, grad):
    """(d_twiddle, d_in_scale, d_out_scale) of scale_twiddle for the gradient `grad` of its result."""
    head = _scale_args(twiddle, in_scale, out_scale)
    assert grad.is_cuda and grad.is_contiguous() and grad.shape == twiddle.shape and grad.dtype == twiddle.dtype
    d_tw = torch.empty_like(twiddle)
    d_in = None if in_scale is None else torch.empty_like(in_scale)
    d_out = None if out_scale is None else torch.empty_like(out_scale)
    _check(lib().bf_butterfly_scale_twiddle_bw(
        *head, int(increasing_stride), _ptr(twiddle),
        None if in_scale is None else _ptr(in_scale), 0 if in_scale is None else in_scale.numel(),
        None if out_scale is None else _ptr(out_scale), 0 if out_scale is None else out_scale.numel(),
        _ptr(grad), _ptr(d_tw), None if d_in is None else _ptr(d_in), None if d_out is None else _ptr(d_out),
        _stream()))
    return d_tw, d_in, d_out


def _table(t, n):
    if t is None:
        return None
    assert t.is_cuda and t.dtype == torch.int32 and t.is_contiguous() and tuple(t.shape) == (n,)
    return _ptr(t)


def multiply_perm_fw(twiddle, input, in_perm, out_index, bias, increasing_stride, output_size=None):
    """Forward between two column permutations (int32 tables of n entries or None):
    u[c] = input[in_perm[c]], output[out_index[c]] = multiply(u)[c] + bias[c]."""
    assert twiddle.is_contiguous() and twiddle.is_cuda and input.is_cuda
    nb, log_n = twiddle.shape[1], twiddle.shape[2]
    n = 1 << log_n
    O = n if output_size is None else output_size
    p = make_problem(input, log_n, nb, increasing_stride, O)
    out = torch.empty(input.shape[0], input.shape[1], O, dtype=input.dtype, device=input.device)
    p.output_stride = _strides(out)
    nbytes = _size(lib().bf_butterfly_multiply_fw_workspace_bytes(ctypes.byref(p)))
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=input.device)
    _check(lib().bf_butterfly_multiply_perm_fw(ctypes.byref(p), _ptr(twiddle), _ptr(input), _table(in_perm, n),
                                               _table(out_index, n), None if bias is None else _ptr(bias),
                                               _ptr(out), _ptr(ws), nbytes, _stream()))
    return out


def multiply_perm_bw(twiddle, input, grad, in_perm, out_index, increasing_stride, with_bias=False):
    """Backward of multiply_perm_fw.  Returns (d_twiddle, d_input, d_bias or None)."""
    assert twiddle.is_contiguous() and twiddle.is_cuda and input.is_cuda and grad.is_cuda
    nb, log_n = twiddle.shape[1], twiddle.shape[2]
    n = 1 << log_n
    p = make_problem(input, log_n, nb, increasing_stride, grad.shape[2])
    p.output_stride = _strides(grad)
    d_twiddle = torch.empty_like(twiddle)
    d_input = torch.empty(input.shape, dtype=input.dtype, device=input.device)
    d_bias = torch.empty(grad.shape[1], grad.shape[2], dtype=grad.dtype, device=grad.device) if with_bias else None
    p.d_input_stride = _strides(d_input)
    size_fn = lib().bf_butterfly_multiply_bias_bw_workspace_bytes if with_bias \
        else lib().bf_butterfly_multiply_bw_workspace_bytes
    nbytes = _size(size_fn(ctypes.byref(p)))
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=input.device)
    _check(lib().bf_butterfly_multiply_perm_bw(ctypes.byref(p), _ptr(twiddle), _ptr(input), _ptr(grad),
                                               _table(in_perm, n), _table(out_index, n), _ptr(d_twiddle),
                                               _ptr(d_input), None if d_bias is None else _ptr(d_bias), _ptr(ws),
                                               nbytes, _stream()))
    return d_twiddle, d_input, d_bias


def multiply_bw(twiddle, input, grad, increasing_stride):
    assert twiddle.is_contiguous() and twiddle.is_cuda and input.is_cuda and grad.is_cuda
    nb, log_n = twiddle.shape[1], twiddle.shape[2]
    p = make_problem(input, log_n, nb, increasing_stride, grad.shape[2])
    p.output_stride = _strides(grad)
    d_twiddle = torch.empty_like(twiddle)
    d_input = torch.empty(input.shape, dtype=input.dtype, device=input.device)
    p.d_input_stride = _strides(d_input)
    nbytes = _size(lib().bf_butterfly_multiply_bw_workspace_bytes(ctypes.byref(p)))
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=input.device)
    _check(lib().bf_butterfly_multiply_bw(ctypes.byref(p), _ptr(twiddle), _ptr(input), _ptr(grad),
                                          _ptr(d_twiddle), _ptr(d_input), _ptr(ws), nbytes, _stream()))
    return d_twiddle, d_input


def multiply_bw_noalloc(twiddle, input, grad, increasing_stride, d_twiddle=None, d_input=None):
    """Backward through the entry point that brings its own scratch area: the caller passes
    operands and results only (results are allocated here when not given)."""
    assert twiddle.is_contiguous() and twiddle.is_cuda and input.is_cuda and grad.is_cuda
    nb, log_n = twiddle.shape[1], twiddle.shape[2]
    p = make_problem(input, log_n, nb, increasing_stride, grad.shape[2])
    p.output_stride = _strides(grad)
    if d_twiddle is None:
        d_twiddle = torch.empty_like(twiddle)
    if d_input is None:
        d_input = torch.empty(input.shape, dtype=input.dtype, device=input.device)
    p.d_input_stride = _strides(d_input)
    _check(lib().bf_butterfly_multiply_bw_noalloc(ctypes.byref(p), _ptr(twiddle), _ptr(input), _ptr(grad),
                                                  _ptr(d_twiddle), _ptr(d_input), _stream()))
    return d_twiddle, d_input


def multiply_fw_bw_saving(twiddle, input, grad, increasing_stride, output_size=None, bias=None, in_perm=None,
                          out_index=None, saved_given=None):
    """Forward that leaves the backward's intermediate activations behind, then the backward that
    reads them.  Returns (output, d_twiddle, d_input, d_bias or None), or None when the problem
    saves nothing.  saved_given: size to declare for the saved area to the backward (tests of the
    size check; default: its real size)."""
    assert twiddle.is_contiguous() and twiddle.is_cuda and input.is_cuda and grad.is_cuda
    nb, log_n = twiddle.shape[1], twiddle.shape[2]
    n = 1 << log_n
    O = n if output_size is None else output_size
    p = make_problem(input, log_n, nb, increasing_stride, O)
    out = torch.empty(input.shape[0], input.shape[1], O, dtype=input.dtype, device=input.device)
    p.output_stride = _strides(out)
    d_input = torch.empty(input.shape, dtype=input.dtype, device=input.device)
    p.d_input_stride = _strides(d_input)
    nsaved = _size(lib().bf_butterfly_multiply_saved_bytes(ctypes.byref(p)))
    if nsaved == 0:
        return None
    saved = torch.empty(nsaved, dtype=torch.uint8, device=input.device)
    _check(lib().bf_butterfly_multiply_fw_saving(ctypes.byref(p), _ptr(twiddle), _ptr(input),
                                                 None if bias is None else _ptr(bias), _table(in_perm, n),
                                                 _table(out_index, n), _ptr(out), _ptr(saved), nsaved, _stream()))
    assert tuple(grad.shape) == tuple(out.shape)
    p.output_stride = _strides(grad)
    d_twiddle = torch.empty_like(twiddle)
    d_bias = None if bias is None else torch.empty_like(bias)
    nbytes = _size(lib().bf_butterfly_multiply_bw_saved_workspace_bytes(ctypes.byref(p), int(bias is not None)))
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=input.device)
    _check(lib().bf_butterfly_multiply_bw_saved(ctypes.byref(p), _ptr(twiddle), _ptr(input), _ptr(grad), _ptr(saved),
                                                saved.numel() if saved_given is None else saved_given,
                                                _table(in_perm, n), _table(out_index, n), _ptr(d_twiddle), _ptr(d_input),
                                                None if d_bias is None else _ptr(d_bias), _ptr(ws), nbytes, _stream()))
    return out, d_twiddle, d_input, d_bias


def multiply_base4_fw(twiddle4, twiddle2, input, increasing_stride, output_size=None):
    assert twiddle4.is_contiguous() and twiddle2.is_contiguous()
    nb = twiddle4.shape[1]
    log_n = twiddle4.shape[2] * 2 + twiddle2.shape[2]
    n = 1 << log_n
    O = n if output_size is None else output_size
    p = make_problem(input, log_n, nb, increasing_stride, O)
    out = torch.empty(input.shape[0], input.shape[1], O, dtype=input.dtype, device=input.device)
    p.output_stride = _strides(out)
    nbytes = _size(lib().bf_butterfly_multiply_base4_fw_workspace_bytes(ctypes.byref(p)))
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=input.device)
    _check(lib().bf_butterfly_multiply_base4_fw(ctypes.byref(p), _ptr(twiddle4), _ptr(twiddle2),
                                                _ptr(input), _ptr(out), _ptr(ws), nbytes, _stream()))
    return out


def multiply_base4_bw(twiddle4, twiddle2, input, grad, increasing_stride):
    assert twiddle4.is_contiguous() and twiddle2.is_contiguous()
    nb = twiddle4.shape[1]
    log_n = twiddle4.shape[2] * 2 + twiddle2.shape[2]
    p = make_problem(input, log_n, nb, increasing_stride, grad.shape[2])
    p.output_stride = _strides(grad)
    d4, d2 = torch.empty_like(twiddle4), torch.empty_like(twiddle2)
    d_input = torch.empty(input.shape, dtype=input.dtype, device=input.device)
    p.d_input_stride = _strides(d_input)
    nbytes = _size(lib().bf_butterfly_multiply_base4_bw_workspace_bytes(ctypes.byref(p)))
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=input.device)
    _check(lib().bf_butterfly_multiply_base4_bw(ctypes.byref(p), _ptr(twiddle4), _ptr(twiddle2), _ptr(input),
                                                _ptr(grad), _ptr(d4), _ptr(d2), _ptr(d_input), _ptr(ws),
                                                nbytes, _stream()))
    return d4, d2, d_input


def multiply_base4_fw_bw_saving(twiddle4, twiddle2, input, grad, increasing_stride, output_size=None):
    """Base-4 forward that leaves the backward's intermediate activations behind, then the
    backward that reads them.  Returns (output, d_twiddle4, d_twiddle2, d_input), or None when
    the problem saves nothing."""
    assert twiddle4.is_contiguous() and twiddle2.is_contiguous()
    nb = twiddle4.shape[1]
    log_n = twiddle4.shape[2] * 2 + twiddle2.shape[2]
    n = 1 << log_n
    O = n if output_size is None else output_size
    p = make_problem(input, log_n, nb, increasing_stride, O)
    out = torch.empty(input.shape[0], input.shape[1], O, dtype=input.dtype, device=input.device)
    p.output_stride = _strides(out)
    d_input = torch.empty(input.shape, dtype=input.dtype, device=input.device)
    p.d_input_stride = _strides(d_input)
    nsaved = _size(lib().bf_butterfly_multiply_base4_saved_bytes(ctypes.byref(p)))
    if nsaved == 0:
        return None
    saved = torch.empty(nsaved, dtype=torch.uint8, device=input.device)
    _check(lib().bf_butterfly_multiply_base4_fw_saving(ctypes.byref(p), _ptr(twiddle4), _ptr(twiddle2), _ptr(input),
                                                       _ptr(out), _ptr(saved), nsaved, _stream()))
    assert tuple(grad.shape) == tuple(out.shape)
    p.output_stride = _strides(grad)
    d4, d2 = torch.empty_like(twiddle4), torch.empty_like(twiddle2)
    nbytes = _size(lib().bf_butterfly_multiply_base4_bw_saved_workspace_bytes(ctypes.byref(p)))
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=input.device)
    _check(lib().bf_butterfly_multiply_base4_bw_saved(ctypes.byref(p), _ptr(twiddle4), _ptr(twiddle2), _ptr(input),
                                                      _ptr(grad), _ptr(saved), saved.numel(), _ptr(d4), _ptr(d2),
                                                      _ptr(d_input),
                                                      _ptr(ws), nbytes, _stream()))
    return out, d4, d2, d_input
