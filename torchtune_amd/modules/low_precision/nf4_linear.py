"""``FrozenNF4Linear``: an ``nn.Linear`` whose weight is a frozen NF4 tensor.

Drop-in for ``torchtune.modules.low_precision.FrozenNF4Linear``
(``torchtune/modules/low_precision/nf4_linear.py:16-70``): same constructor, same parameter layout (one
``weight`` parameter holding an ``NF4Tensor``, optional frozen ``bias``), forward through ``linear_nf4``.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn

from ...nf4_tensor import linear_nf4, to_nf4


class FrozenNF4Linear(nn.Linear):
    def __init__(
        self,
        in_dim: int,
        out_dim: int,
        bias: bool = False,
        device: Optional[torch.device] = None,
        dtype: Optional[torch.dtype] = None,
        **quantization_kwargs,
    ):
        super().__init__(in_dim, out_dim, bias=bias, device=device, dtype=dtype)
        for p in (self.weight, self.bias):
            if p is not None:
                p.requires_grad_(False)
        packed = nn.Parameter(to_nf4(self.weight, **quantization_kwargs), requires_grad=False)
        # swap in place so the NF4 tensor is what .parameters() / state_dict() report
        torch.utils.swap_tensors(self.weight, packed)

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        y = linear_nf4(input=input, weight=self.weight)
        return y if self.bias is None else y + self.bias
