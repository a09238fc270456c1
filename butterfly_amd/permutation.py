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

    def to_butterfly(self, complex=False, increasing_stride=False):
        """A two-block Butterfly with the same effect (torch_butterfly/permutation.py:77-78)."""
        return perm2butterfly(self.permutation, complex, increasing_stride)

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
    """0/1 matrix M of the permutation vector p.  left=False (right-multiplication format):
    M[p[i], i] = 1, so the row vector x M equals x[p]; left=True gives the transpose, for which
    M x equals x[p] (reference: torch_butterfly/permutation.py:98-108)."""
    p = np.asarray(p)
    m = np.zeros((p.size, p.size), dtype=np.int64)
    m[p, np.arange(p.size)] = 1
    return m.T if left else m


def perm_mat_to_vec(m, left=False):
    """Inverse of perm_vec_to_mat (reference: torch_butterfly/permutation.py:111-118)."""
    m = np.asarray(m)
    return np.argmax(m if left else m.T, axis=1)


def is_2x2_block_diag(mat):
    """True when each of the four quadrants of the (even-sized, square) matrix is diagonal, i.e.
    entry (i, j) vanishes unless i - j is a multiple of half the size: a 2 x 2 grid of diagonal
    blocks, the shape of one butterfly factor over the whole matrix
    (reference: torch_butterfly/permutation.py:121-130)."""
    mat = np.asarray(mat)
    n = mat.shape[0]
    if mat.shape != (n, n) or n % 2:
        return False
    i, j = np.indices((n, n))
    return not np.any(mat[(i - j) % (n // 2) != 0])


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


def half_balance(v, return_swap_locations=False):
    """Swaps between positions i and i + n/2 after which the first half of the vector v (values
    distinct modulo n, n even) holds every residue modulo n/2 once, and so does the second half.
    Returns ``(perm, v[perm])`` with perm the product of the swaps, or ``(low positions of
    the swapped pairs, v[perm])``.

    Two positions that hold the same residue must end in different halves, and so must the
    two positions of a pair (i, i + n/2): following "same residue" and "same pair" alternately
    from any position walks a closed loop of even length, and keeping the first element where
    it is fixes every other choice on the loop.  (The reference builds the same loops as an
    edge-oriented graph, torch_butterfly/permutation.py:176-228; which of the two valid
    settings a loop gets is not part of the contract.)"""
    v = np.asarray(v)
    n = v.size
    if n % 2:
        raise ValueError("the vector must have even length")
    nh = n // 2
    residue = v % nh
    order = np.argsort(residue, kind="stable")          # positions by residue: two per residue
    if not np.array_equal(residue[order], np.repeat(np.arange(nh), 2)):
        raise ValueError("every residue modulo n/2 must occur exactly twice")
    rival = np.empty(n, dtype=np.int64)
    rival[order[0::2]] = order[1::2]
    rival[order[1::2]] = order[0::2]
    swapped = np.zeros(nh, dtype=bool)
    seen = np.zeros(n, dtype=bool)
    for start in range(n):
        if seen[start]:
            continue
        pos = start
        half = int(pos >= nh)                           # the half this element ends in: it stays put
        while not seen[pos]:
            seen[pos] = True
            other = rival[pos]                          # same residue: must end in the other half
            seen[other] = True
            swapped[other % nh] = (int(other >= nh) == half)
            pos = (other + nh) % n                      # its pair partner ends in `half` again
    low = np.flatnonzero(swapped)
    perm = np.arange(n)
    perm[low], perm[low + nh] = low + nh, low
    return (low.tolist() if return_swap_locations else perm), v[perm]


def modular_balance(v):
    """The swaps that make the permutation vector v modular-balanced, level by level: blocks of
    n, n/2, ..., 2 consecutive positions are half-balanced in turn.  Returns ``(perms, w)`` with
    ``w = v[perms[0]][perms[1]]...`` and w modular-balanced
    (reference: torch_butterfly/permutation.py:231-252)."""
    v = np.asarray(v)
    n = v.size
    perms = []
    t = n
    while t >= 2:
        level = np.concatenate([half_balance(v[base:base + t])[0] + base for base in range(0, n, t)])
        v = v[level]
        perms.append(level)
        t //= 2
    return perms, v


def is_modular_balanced(perm):
    """True when every aligned block of j = 2, 4, ..., n consecutive entries of the permutation
    (vector, or matrix in right-multiplication format) holds j different residues modulo j
    (reference: torch_butterfly/permutation.py:255-269)."""
    perm = np.asarray(perm)
    if perm.ndim > 1:
        perm = perm_mat_to_vec(perm)
    n = perm.size
    log_n = int(n).bit_length() - 1
    if n != 1 << log_n:
        raise ValueError("the size must be a power of 2")
    for k in range(1, log_n + 1):
        j = 1 << k
        residues = np.sort((perm % j).reshape(n // j, j), axis=1)
        if not np.array_equal(residues, np.broadcast_to(np.arange(j), (n // j, j))):
            return False
    return True


def _balanced_factor_vectors(w):
    """w modular-balanced (right-multiplication vector, x L = x[w]): vectors f_n, f_{n/2}, ...,
    f_2 with w = f_n[f_{n/2}[...[f_2]]], f_k moving entries by 0 or +-k/2 inside blocks of k."""
    n = w.size
    if n == 2:
        return [w.copy()]
    nh = n // 2
    inner = np.concatenate((w[:nh] % nh, w[nh:] % nh + nh))    # what is left inside the two halves
    outer = w[invert(inner)]                                   # w = outer[inner]
    first = _balanced_factor_vectors(inner[:nh])
    second = _balanced_factor_vectors(inner[nh:] - nh)
    return [outer] + [np.concatenate((a, b + nh)) for a, b in zip(first, second)]


def modular_balanced_to_butterfly_factor(L):
    """Butterfly factors (permutation matrices in right-multiplication format, block sizes
    n, n/2, ..., 2) whose product in that order is the modular-balanced permutation L (vector or
    matrix in right-multiplication format; reference: torch_butterfly/permutation.py:272-301)."""
    L = np.asarray(L)
    w = L if L.ndim == 1 else perm_mat_to_vec(L)
    if not is_modular_balanced(w):
        raise ValueError("the permutation is not modular-balanced")
    return [perm_vec_to_mat(f) for f in _balanced_factor_vectors(w.astype(np.int64))]


def _butterfly_from_gathers(block0, block1, n, size, complex):
    """Two-block Butterfly (decreasing stride first) from its factors given as gathers
    (x -> x[f]): block0 with block sizes n, n/2, ..., 2 and block1 with 2, 4, ..., n."""
    from .butterfly import Butterfly  # (butterfly.py does not import this module)
    log_n = n.bit_length() - 1
    planes = []
    for factors, sizes in ((block0, range(log_n, 0, -1)), (block1, range(1, log_n + 1))):
        planes.append(torch.stack([matrix_to_butterfly_factor(perm_vec_to_mat(f, left=True), log_k, pytorch_format=True)
                                   for f, log_k in zip(factors, sizes)]))
    dtype = torch.get_default_dtype()
    if complex:
        from .complex_utils import real_dtype_to_complex
        dtype = real_dtype_to_complex[dtype]
    twiddle = torch.stack(planes).unsqueeze(0).to(dtype)
    b = Butterfly(n, n, bias=False, complex=complex, increasing_stride=False, init=twiddle, nblocks=2)
    b.in_size = b.out_size = size
    return b


def _padded_permutation(v):
    if isinstance(v, torch.Tensor):
        v = v.detach().cpu().numpy()
    v = np.asarray(v, dtype=np.int64)
    size = v.size
    if size < 2:
        raise ValueError("the permutation must have at least 2 elements")
    if not np.array_equal(np.sort(v), np.arange(size)):
        raise ValueError("v is not a permutation")
    n = 1 << int(size - 1).bit_length()
    return np.concatenate((v, np.arange(size, n, dtype=np.int64))), size, n


def _to_increasing_stride(b, size):
    """The decreasing-stride Butterfly of br[v[br]] read with increasing stride and its pairs
    in bit-reversed order is a Butterfly of v (torch_butterfly/permutation.py:322-330)."""
    from .butterfly import Butterfly
    n = b.twiddle.shape[3] * 2
    pairs = bitreversal_permutation(n // 2, pytorch_format=True)
    out = Butterfly(n, n, bias=False, complex=b.twiddle.is_complex(), increasing_stride=True,
                    init=b.twiddle.detach()[:, :, :, pairs].clone(), nblocks=2)
    out.in_size = out.out_size = size
    return out


def perm2butterfly_slow(v, complex=False, increasing_stride=False):
    """``b(x) == x[..., v]`` as perm2butterfly, built the way the existence proof goes: the
    level-by-level swaps of ``modular_balance`` are the first block, the factors of the
    modular-balanced rest the second (reference: torch_butterfly/permutation.py:304-348)."""
    full, size, n = _padded_permutation(v)
    if increasing_stride:
        br = bitreversal_permutation(n)
        return _to_increasing_stride(perm2butterfly_slow(br[full[br]], complex, False), size)
    # invert(full) = w[s_last[...[s_first]]] with s the swaps, so
    # x[full] = x[s_first]...[s_last][invert(w)] and invert(w) = invert(f_2)[...[invert(f_n)]].
    swaps, w = modular_balance(invert(full))
    block1 = [invert(f) for f in reversed(_balanced_factor_vectors(w))]
    return _butterfly_from_gathers(swaps, block1, n, size, complex)


def swap_locations_to_twiddle_factor(n, swap_locations):
    """(n/2, 2, 2) factor of straight switches, crossed at the given pair indices."""
    twiddle = torch.eye(2).repeat(n // 2, 1, 1)
    twiddle[torch.as_tensor(np.asarray(swap_locations, dtype=np.int64))] = torch.tensor([[0.0, 1.0], [1.0, 0.0]])
    return twiddle


def outer_twiddle_factors(v):
    """One level of the permutation-to-butterfly recursion for a batch of permutations v
    (batch, size), left-multiplication format: the switch factor applied first
    (batch * size/2, 2, 2), the one applied last (same shape), and the 2 * batch permutations
    of size/2 left between them (reference: torch_butterfly/permutation.py:358-392)."""
    v = np.asarray(v)
    batch, size = v.shape
    if size < 2:
        raise ValueError("size must be at least 2")
    half = size // 2
    first, rest = [], []
    for row in v:
        low, balanced = half_balance(invert(row), return_swap_locations=True)
        first.append(swap_locations_to_twiddle_factor(size, low))
        rest.append(invert(balanced))
    rest = np.stack(rest)                                     # rest[b][c]: source of output c
    crossed = rest[:, :half] >= half                          # output pair c takes its low element from the top half
    rows, cols = np.nonzero(crossed)
    last = swap_locations_to_twiddle_factor(batch * size, rows * half + cols)
    lo, hi = rest[:, :half].copy(), rest[:, half:].copy()
    lo[crossed], hi[crossed] = rest[:, half:][crossed], rest[:, :half][crossed]
    inner = np.concatenate((lo, hi), axis=1) % half
    inner = inner.reshape(batch * 2, half)
    if not np.array_equal(np.sort(inner, axis=1), np.broadcast_to(np.arange(half), inner.shape)):
        raise AssertionError("the inner vectors are not permutations")
    return torch.cat(first), last, inner


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
