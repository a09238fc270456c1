"""The legacy ``butterfly`` package's learnable permutation: a product of relaxed
permutation factors, each a convex mix of "leave as is" with a fixed shuffle.

Counterpart of the reference's butterfly/permutation.py (``Permutation``, ``FixedPermutation``,
``PermutationFactor``) and of ``permutation_mult`` / ``permutation_mult_single`` from
butterfly/permutation_multiply.py:18-52, 173-221, with the same names, argument order,
parameter names and shapes.  A factor is elementwise work on the activations with three
scalars per step, not a butterfly multiply, so it is written with tensor views and ``lerp``
and runs wherever its input lives; autograd supplies the gradients.

One factor acts on groups of ``w = 2 * stride`` consecutive elements, halves ``a`` in {0, 1},
position ``j`` < stride inside a half, with probabilities ``(p, q0, q1)``:

    dealt[a * stride + j] = (1 - p)  * x[a * stride + j]     + p  * x[2 j + a]
    out  [a * stride + j] = (1 - qa) * dealt[a * stride + j] + qa * dealt[a * stride + stride - 1 - j]

i.e. with weight ``p`` the even elements are dealt to the first half and the odd ones to the
second, then each half is reversed with its own weight.  ``prob[k - 1]`` belongs to
``stride = 2^k`` whatever the order of application.  Complex data are real tensors with a
trailing dimension of 2.
"""
import torch
from torch import nn


def _log2(n):
    m = int(n).bit_length() - 1
    if n < 1 or n != 1 << m:
        raise ValueError("size must be a power of 2")
    return m


def _factor(x, prob, stride):
    """One relaxed permutation factor on x (batch, n) or (batch, n, 2); prob (3,)."""
    batch, n = x.shape[:2]
    tail = x.shape[2:]
    groups = n // (2 * stride)
    halves = x.reshape(batch, groups, 2, stride, *tail)
    dealt_src = x.reshape(batch, groups, stride, 2, *tail).transpose(2, 3)
    dealt = torch.lerp(halves, dealt_src, prob[0])
    q = prob[1:].reshape(2, 1, *([1] * len(tail)))
    return torch.lerp(dealt, dealt.flip(3), q).reshape(x.shape)


def _check(prob, input):
    if input.dim() not in (2, 3) or (input.dim() == 3 and input.shape[2] != 2):
        raise ValueError("input must be (batch, n) if real or (batch, n, 2) if complex")
    return _log2(input.shape[1])


def permutation_mult(prob, input, increasing_stride=False, return_intermediates=False):
    """Apply the factors with strides 2, 4, ..., 2^nsteps (that order when
    ``increasing_stride``, the reverse otherwise); prob (nsteps, 3), nsteps <= log2(n) - 1.
    With ``return_intermediates`` the input and the result of every step, stacked."""
    m = _check(prob, input)
    if prob.dim() != 2 or prob.shape[1] != 3 or prob.shape[0] > max(m - 1, 0):
        raise ValueError("prob must be (nsteps, 3) with nsteps <= log2(n) - 1")
    order = range(1, prob.shape[0] + 1)
    out = input.contiguous()
    trail = [out]
    for k in (order if increasing_stride else reversed(order)):
        out = _factor(out, prob[k - 1], 1 << k)
        trail.append(out)
    return torch.stack(trail) if return_intermediates else out


def permutation_mult_single(prob, input):
    """The one factor whose group is the whole row (stride n / 2); prob (3,)."""
    m = _check(prob, input)
    if prob.shape != (3,) or m < 1:
        raise ValueError("prob must be (3,) and n at least 2")
    return _factor(input.contiguous(), prob, input.shape[1] // 2)


# Names the reference exports for its two implementations of the same function.
permutation_mult_torch = permutation_mult
permutation_mult_factors = permutation_mult
permutation_mult_single_factor = permutation_mult_single
permutation_mult_single_factor_torch = permutation_mult_single


class Permutation(nn.Module):
    """Product of log2(size) - 1 relaxed permutation factors with learnable logits
    (``logit``: (log2(size) - 1, 3), or (3,) shared by all factors when ``share_logit``);
    probabilities are their sigmoids (butterfly/permutation.py:9-55)."""

    def __init__(self, size, share_logit=False, increasing_stride=False):
        super().__init__()
        self.size = size
        self.nsteps = _log2(size) - 1
        self.share_logit = share_logit
        self.increasing_stride = increasing_stride
        self.logit = nn.Parameter(torch.randn(3) if share_logit else torch.randn(self.nsteps, 3))

    def _prob(self, logit):
        prob = torch.sigmoid(logit)
        return prob.unsqueeze(0).expand(self.nsteps, 3) if self.share_logit else prob

    def forward(self, input):
        """input, output: (batch, size) if real or (batch, size, 2) if complex."""
        return permutation_mult(self._prob(self.logit), input, increasing_stride=self.increasing_stride)

    def argmax(self):
        """(size,) int64: the permutation the factors make when every probability is rounded,
        as the gather ``output = input[:, p]``."""
        with torch.no_grad():
            prob = self._prob(self.logit).round()
            index = torch.arange(self.size, dtype=prob.dtype, device=prob.device).unsqueeze(0)
            moved = permutation_mult(prob, index, increasing_stride=self.increasing_stride)
        return moved.squeeze(0).round().long()

    def extra_repr(self):
        return f"size={self.size}, share_logit={self.share_logit}, increasing_stride={self.increasing_stride}"


class FixedPermutation(nn.Module):
    """``output = input[:, permutation]``; holds the argmax of a ``Permutation``
    (butterfly/permutation.py:58-76)."""

    def __init__(self, permutation):
        super().__init__()
        self.register_buffer('permutation', permutation)

    def forward(self, input):
        return input[:, self.permutation]


class PermutationFactor(nn.Module):
    """A single factor over the whole row, ``logit`` (3,) (butterfly/permutation.py:79-113)."""

    def __init__(self, size):
        super().__init__()
        self.size = size
        if _log2(size) < 1:
            raise ValueError("size must be at least 2")
        self.logit = nn.Parameter(torch.randn(3))

    def forward(self, input):
        return permutation_mult_single(torch.sigmoid(self.logit), input)

    def argmax(self):
        with torch.no_grad():
            prob = torch.sigmoid(self.logit).round()
            index = torch.arange(self.size, dtype=prob.dtype, device=prob.device).unsqueeze(0)
            return permutation_mult_single(prob, index).squeeze(0).round().long()

    def extra_repr(self):
        return f"size={self.size}"
