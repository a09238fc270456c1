"""``ButterflyBase4``: the same layer as ``Butterfly`` with stage pairs pre-fused into 4x4
factors (parameters ``twiddle4`` / ``twiddle2``), evaluated by the native base-4 operator.
Mirrors torch_butterfly/butterfly_base4.py:15-72 of the reference."""
import numbers

import torch
from torch import nn

from .butterfly import Butterfly
from .multiply_base4 import butterfly_multiply_base4, twiddle_base2_to_base4


class ButterflyBase4(Butterfly):
    """Arguments as for ``Butterfly``; ``init`` may also be a ``(twiddle4, twiddle2)`` pair."""

    def __init__(self, *args, **kwargs):
        init = kwargs.get("init", None)
        pair = (isinstance(init, tuple) and len(init) == 2
                and all(isinstance(t, torch.Tensor) for t in init))
        if pair:
            twiddle4, twiddle2 = init[0].clone(), init[1].clone()
            kwargs["init"] = "empty"
            super().__init__(*args, **kwargs)
        else:
            super().__init__(*args, **kwargs)
            with torch.no_grad():
                twiddle4, twiddle2 = twiddle_base2_to_base4(self.twiddle, self.increasing_stride)
                twiddle4, twiddle2 = twiddle4.clone(), twiddle2.clone()
        del self.twiddle
        self.twiddle4 = nn.Parameter(twiddle4)
        self.twiddle2 = nn.Parameter(twiddle2)
        self.twiddle4._is_structured = True
        self.twiddle2._is_structured = True

    def forward(self, input):
        x = self.pre_process(input)
        output_size = self.out_size if self.nstacks == 1 else None
        x = butterfly_multiply_base4(self.twiddle4, self.twiddle2, x, self.increasing_stride,
                                     output_size)
        return self.post_process(input, x)

    def __imul__(self, scale):
        if not isinstance(scale, numbers.Number) or scale < 0:
            raise ValueError("scale must be a non-negative number")
        per_stage = scale ** (1.0 / (self.nblocks * self.log_n))
        self.twiddle4 *= per_stage ** 2
        self.twiddle2 *= per_stage
        return self
