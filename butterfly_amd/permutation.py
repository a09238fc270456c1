"""Fixed permutations on the multiply path: the FFT bit reversal, a module that applies a
stored permutation (reference: torch_butterfly/permutation.py:14-30,55-78) and a Sequential
that folds such modules into the neighbouring Butterfly's kernels."""
import numpy as np
import torch
from torch import nn

from .complex_utils import index_last_dim


def bitreversal_permutation(n, pytorch_format=False):
    """perm[i] = i with its log2(n) bits reversed."""
    log_n = int(n).bit_length() - 1
    if n != 1 << log_n:
        raise ValueError("n must be a power of 2")
    idx = np.arange(n)
    perm = np.zeros(n, dtype=np.int64)
    for bit in range(log_n):
        perm |= ((idx >> bit) & 1) << (log_n - 1 - bit)
    return torch.from_numpy(perm) if pytorch_format else perm


def invert(perm):
    """Inverse permutation (numpy array or tensor)."""
    if isinstance(perm, torch.Tensor):
        inv = torch.empty_like(perm)
        inv[perm] = torch.arange(perm.numel(), dtype=perm.dtype, device=perm.device)
        return inv
    inv = np.empty_like(perm)
    inv[perm] = np.arange(perm.size)
    return inv


class FixedPermutation(nn.Module):
    """output[..., i] = input[..., permutation[i]]."""

    def __init__(self, permutation: torch.Tensor) -> None:
        super().__init__()
        self.register_buffer("permutation", permutation)
        self._tables = {}

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        return index_last_dim(input, self.permutation)

    def column_table(self, n: int, scatter: bool) -> torch.Tensor:
        """The permutation as the int32 table of n entries that the multiply operators fold
        into their first read (scatter False: entry c = permutation[c]) or their last write
        (scatter True: the inverse, entry permutation[i] = i); entries past the permutation's
        length are fixed points.  Cached until the buffer changes."""
        p = self.permutation
        key = (n, scatter, p.device, p.data_ptr(), p._version)
        table = self._tables.get(key)
        if table is None:
            if p.dim() != 1 or p.numel() > n:
                raise ValueError("the permutation must be a vector of at most n entries")
            full = torch.arange(n, dtype=torch.int64, device=p.device)
            full[:p.numel()] = p
            table = (invert(full) if scatter else full).to(torch.int32)
            if len(self._tables) >= 4:
                self._tables.clear()
            self._tables[key] = table
        return table


class FusedSequential(nn.Sequential):
    """nn.Sequential (same children, indexing and state) whose forward folds what stands
    directly around a Butterfly into that layer's own call: a FixedPermutation in front of or
    behind it becomes part of the kernels' first read / last write, and a Diagonal between that
    permutation and the layer (or alone next to the layer) is multiplied into the layer's first /
    last factor, so neither costs a pass of its own over the activations.  The accepted
    patterns are [FixedPermutation] [Diagonal] Butterfly [Diagonal] [FixedPermutation]; any
    other sequence of children runs one after the other as usual."""

    def forward(self, input):
        from .butterfly import Butterfly, ButterflyBmm  # (butterfly.py does not import this module)
        from .diagonal import Diagonal
        mods = list(self)

        def is_layer(m):
            return isinstance(m, Butterfly) and not isinstance(m, ButterflyBmm)

        def is_perm(m, size):
            return isinstance(m, FixedPermutation) and m.permutation.dim() == 1 and m.permutation.numel() == size

        def is_scale(m, size, layer):
            return (isinstance(m, Diagonal) and m.diagonal.dim() == 1 and m.diagonal.numel() == size
                    and (layer.complex or not m.diagonal.is_complex()))

        i = 0
        while i < len(mods):
            # the layer that a permutation and / or a diagonal at position i would lead to
            j = i
            while j < len(mods) and j - i < 2 and isinstance(mods[j], (FixedPermutation, Diagonal)):
                j += 1
            layer = mods[j] if j < len(mods) and is_layer(mods[j]) else None
            front = scale_in = None
            if layer is not None and input.is_cuda and input.is_complex() == layer.complex:
                lead = mods[i:j]
                if len(lead) == 2 and is_perm(lead[0], layer.in_size) and is_scale(lead[1], layer.in_size, layer):
                    front, scale_in = lead
                elif len(lead) == 1 and is_perm(lead[0], layer.in_size):
                    front = lead[0]
                elif len(lead) == 1 and is_scale(lead[0], layer.in_size, layer):
                    scale_in = lead[0]
                elif lead:
                    layer = None
            else:
                layer = None if j > i else layer
            if layer is None or not input.is_cuda or input.is_complex() != layer.complex:
                input = mods[i](input)
                i += 1
                continue
            i = j + 1
            back = scale_out = None
            if i < len(mods) and layer.bias is None and is_scale(mods[i], layer.out_size, layer):
                scale_out = mods[i]
                i += 1
            if i < len(mods) and layer.nstacks == 1 and is_perm(mods[i], layer.out_size):
                back = mods[i]
                i += 1
            n = 1 << layer.log_n
            input = layer(input, in_perm=None if front is None else front.column_table(n, False),
                          out_index=None if back is None else back.column_table(n, True),
                          in_scale=None if scale_in is None else scale_in.diagonal,
                          out_scale=None if scale_out is None else scale_out.diagonal)
        return input


def wavelet_permutation(n, pytorch_format=False):
    """Order of the in-place multilevel Haar transform's outputs: position 0 (the coarsest
    average), then the positions whose lowest set bit is log2(n) - 1, log2(n) - 2, ..., 0, each
    group ascending -- [0, 4, 2, 6, 1, 3, 5, 7] for n = 8
    (reference: torch_butterfly/permutation.py:33-52)."""
    log_n = int(n).bit_length() - 1
    if n != 1 << log_n:
        raise ValueError("n must be a power of 2")
    groups = [np.zeros(1, dtype=np.int64)]
    for bit in range(log_n - 1, -1, -1):
        groups.append(np.arange(1 << bit, n, 2 << bit, dtype=np.int64))
    perm = np.concatenate(groups)
    return torch.from_numpy(perm) if pytorch_format else perm


def perm_vec_to_mat(p, left=False):
    """0/1 matrix of the permutation vector p: (M x)[i] = x[p[i]] (left=False), i.e.
    M[i, p[i]] = 1; left=True gives the transpose (x M convention)."""
    p = np.asarray(p)
    m = np.zeros((p.size, p.size), dtype=np.int64)
    m[np.arange(p.size), p] = 1
    return m.T if left else m


def perm_mat_to_vec(m, left=False):
    """Inverse of perm_vec_to_mat."""
    m = np.asarray(m)
    return np.argmax(m.T if left else m, axis=1)


def is_2x2_block_diag(mat):
    """True when mat is block diagonal with 2x2 blocks."""
    mat = np.asarray(mat)
    n = mat.shape[0]
    if mat.shape != (n, n) or n % 2:
        return False
    mask = np.kron(np.eye(n // 2, dtype=bool), np.ones((2, 2), dtype=bool))
    return not np.any(mat[~mask])


def is_butterfly_factor(mat, k):
    """True when mat is a butterfly factor of block size k: block diagonal with k x k blocks, each
    of which only couples i with i + k/2 (four diagonal k/2 x k/2 sub-blocks)."""
    mat = np.asarray(mat)
    n = mat.shape[0]
    if mat.shape != (n, n) or n % k or k % 2:
        return False
    i, j = np.indices((n, n))
    allowed = (i // k == j // k) & ((i - j) % (k // 2) == 0)
    return not np.any(mat[~allowed])


def matrix_to_butterfly_factor(mat, log_k, pytorch_format=False, check_input=False):
    """The (n/2, 2, 2) twiddle of the butterfly factor ``mat`` of block size k = 2^log_k: pair
    index i couples positions pos and pos + k/2 with pos = 2 (i - i mod k/2) + i mod k/2."""
    mat = np.asarray(mat)
    n = mat.shape[0]
    k = 1 << log_k
    if check_input and not is_butterfly_factor(mat, k):
        raise ValueError("not a butterfly factor of this block size")
    half = k // 2
    i = np.arange(n // 2)
    low = i % half
    pos = 2 * (i - low) + low
    rows = np.stack((pos, pos + half), -1)                       # (n/2, 2)
    tw = mat[rows[:, :, None], rows[:, None, :]]                 # tw[i, r, c] = mat[rows[i, r], rows[i, c]]
    return torch.from_numpy(np.ascontiguousarray(tw)) if pytorch_format else tw


def _benes_switches(perm, log_n, increasing_stride):
    """Routes ``perm`` (out[d] = in[perm[d]]) through the 2 log_n stages of a two-block
    butterfly whose factors are straight / crossed 2x2 switches (a Benes network: stage j of
    the first block and stage log_n - 1 - j of the second both pair bit b_j = j for increasing
    stride, log_n - 1 - j for decreasing).  Looping algorithm, one level per pass: signals
    sharing an input pair or an output pair of the level's bit take different halves, which
    2-colours every loop; the colours set the two outer switch columns and leave a permutation
    inside each half for the next level.  Returns cross[2][log_n][n/2] booleans."""
    n = 1 << log_n
    cross = np.zeros((2, log_n, n // 2), dtype=bool)
    cur = np.asarray(perm, dtype=np.int64).copy()
    for depth in range(log_n):
        b = depth if increasing_stride else log_n - 1 - depth
        bit = 1 << b
        lowmask = bit - 1

        def pair_index(e):
            return ((e >> (b + 1)) << b) | (e & lowmask)

        if depth == log_n - 1:
            # two positions per sub-network left: one switch does it, the other stays straight
            lo = np.flatnonzero((np.arange(n) & bit) == 0)
            swapped = cur[lo] != lo
            cross[0, depth, pair_index(lo)] = swapped
            break
        inv = np.empty(n, dtype=np.int64)
        inv[cur] = np.arange(n)
        colour = np.full(n, -1, dtype=np.int64)
        for start in range(n):
            if colour[start] >= 0:
                continue
            d = start
            while colour[d] < 0:
                colour[d] = 0
                partner = d ^ bit               # shares the output pair: other half
                colour[partner] = 1
                d = inv[cur[partner] ^ bit]     # shares the input pair with that one: first half again
        src = cur                                # signal d comes from src[d]
        # input switch of the pair of s: crossed when the signal entering at the low position leaves for half 1
        lo_src = np.flatnonzero((src & bit) == 0)            # signals (by destination) whose source has the bit clear
        cross[0, depth, pair_index(src[lo_src])] = colour[lo_src] == 1
        # output switch: crossed when the signal bound for the low position travels in half 1
        lo_dst = np.flatnonzero((np.arange(n) & bit) == 0)
        cross[1, log_n - 1 - depth, pair_index(lo_dst)] = colour[lo_dst] == 1
        # inside the halves: signal d now sits at src with the bit set to its colour and must
        # reach d with the bit set to its colour
        d_all = np.arange(n)
        inner_dst = (d_all & ~bit) | (colour * bit)
        inner_src = (src & ~bit) | (colour * bit)
        nxt = np.empty(n, dtype=np.int64)
        nxt[inner_dst] = inner_src
        cur = nxt
    return cross


def perm2butterfly(v, complex=False, increasing_stride=False):
    """A two-block Butterfly whose matrix is the permutation v: ``b(x) == x[..., v]``.
    v is padded with fixed points to the next power of 2
    (reference: torch_butterfly/permutation.py:395-433)."""
    from .butterfly import Butterfly  # (butterfly.py does not import this module)
    if isinstance(v, torch.Tensor):
        v = v.detach().cpu().numpy()
    v = np.asarray(v, dtype=np.int64)
    size = v.size
    if size < 2:
        raise ValueError("the permutation must have at least 2 elements")
    if not np.array_equal(np.sort(v), np.arange(size)):
        raise ValueError("v is not a permutation")
    log_n = int(size - 1).bit_length()
    n = 1 << log_n
    full = np.concatenate((v, np.arange(size, n, dtype=np.int64)))
    cross = _benes_switches(full, log_n, increasing_stride)
    dtype = torch.get_default_dtype()
    if complex:
        from .complex_utils import real_dtype_to_complex
        dtype = real_dtype_to_complex[dtype]
    straight = torch.eye(2, dtype=dtype)
    crossed = torch.tensor([[0.0, 1.0], [1.0, 0.0]], dtype=dtype)
    pick = torch.from_numpy(cross).reshape(1, 2, log_n, n // 2, 1, 1)
    twiddle = torch.where(pick, crossed, straight)
    b = Butterfly(n, n, bias=False, complex=complex, increasing_stride=increasing_stride, init=twiddle, nblocks=2)
    b.in_size = size
    b.out_size = size
    return b
