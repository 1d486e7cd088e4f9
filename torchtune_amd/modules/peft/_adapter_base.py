"""What ``LoRALinear`` and ``DoRALinear`` have in common: a frozen base linear (dense or NF4) plus the two low-rank
factors, their initialisation, and the checks that decide whether the fused HIP kernels apply.

Reference behaviour being mirrored: ``torchtune/modules/peft/lora.py:57-126,309-320`` and
``torchtune/modules/peft/dora.py:50-111`` (constructor arguments, attribute and parameter names, the ``ValueError`` for
quantisation arguments without ``quantize_base``, Kaiming-uniform ``lora_a``, zero ``lora_b``).
"""
from __future__ import annotations

import math
from typing import Optional, Union

import torch
import torch.nn.functional as F
from torch import nn

from ... import ops
from ...nf4_tensor import NF4Tensor, _fused_ok, linear_nf4, to_nf4
from ..low_precision import _register_nf4_dispatch_ops  # noqa: F401  (clone override must be active)


def _lora_a_init_params(x: nn.Linear) -> None:
    """Kaiming-uniform, a = sqrt(5)."""
    nn.init.kaiming_uniform_(x.weight, a=math.sqrt(5))


def _lora_b_init_params(x: nn.Linear) -> None:
    """Zeros: the adapter starts as a no-op."""
    nn.init.zeros_(x.weight)


class LowRankAdapterLinear(nn.Module):
    """Base of the adapter layers.  Owns ``weight`` (dense or ``NF4Tensor``), ``bias``, ``dropout``, ``lora_a``,
    ``lora_b`` and the ``disabled`` switch; subclasses add their own attributes and ``forward``."""

    def _build(self, in_dim: int, out_dim: int, rank: int, dropout: float, use_bias: bool, quantize_base: bool,
               quantization_kwargs: dict) -> None:
        if not quantize_base and any(v for v in quantization_kwargs.values()):
            raise ValueError(
                f"``quantize_base`` is False, but received the following quantization arguments: {quantization_kwargs}"
            )
        self.in_dim = in_dim
        self.out_dim = out_dim
        self.use_bias = use_bias
        self._quantize_base = quantize_base
        self.disabled = False  # True: behave as the frozen base layer alone (the reference policy in DPO)
        dense = nn.Linear(in_features=in_dim, out_features=out_dim, bias=use_bias)
        self.register_parameter(
            "weight", nn.Parameter(to_nf4(dense.weight, **quantization_kwargs) if quantize_base else dense.weight)
        )
        self.register_parameter("bias", nn.Parameter(dense.bias) if use_bias else None)
        self.dropout = nn.Dropout(p=dropout) if dropout > 0.0 else nn.Identity()
        self.lora_a = nn.Linear(in_features=in_dim, out_features=rank, bias=False)
        self.lora_b = nn.Linear(in_features=rank, out_features=out_dim, bias=False)

    def to_empty(self, *, device: Optional[Union[str, torch.device, int]], recurse: bool = True):
        self.lora_a.to_empty(device=device, recurse=recurse)
        self.lora_b.to_empty(device=device, recurse=recurse)

    def initialize_parameters(self):
        _lora_a_init_params(self.lora_a)
        _lora_b_init_params(self.lora_b)

    # ---- what the subclasses' forward passes share ---------------------------------------------------
    def _adapter_rank(self) -> int:
        return self.lora_a.weight.shape[0]

    def _dropping(self) -> bool:
        return self.training and isinstance(self.dropout, nn.Dropout) and self.dropout.p > 0.0

    def _nf4_kernels_apply(self, dtype: torch.dtype) -> bool:
        """The base weight is an NF4 tensor the fused bf16 kernels can read, and the factors are bf16."""
        w = self.weight
        rank = self._adapter_rank()
        return (
            isinstance(w, NF4Tensor) and w.is_cuda and w.dim() == 2 and w.block_size == 64 and w.dtype == torch.bfloat16
            and dtype == torch.bfloat16 and rank > 0 and ops.fused_shape_ok(w.shape[0], w.shape[1], rank)
            and self.lora_a.weight.dtype == torch.bfloat16 and self.lora_b.weight.dtype == torch.bfloat16
        )

    def _fused_path(self, x: torch.Tensor) -> bool:
        if not self._quantize_base or x.dtype != torch.bfloat16 or self._dropping():
            return False
        # what depends on the parameters alone is decided once per set of parameter objects (a swapped or re-created
        # parameter is another object): attribute reads on an NF4 tensor subclass cost microseconds each
        w, a, b, bias = self.weight, self.lora_a.weight, self.lora_b.weight, self.bias
        packed = getattr(w, "quantized_data", None)  # the inner tensor object: another one after a move or a rewrap
        memo = self.__dict__.get("_fused_memo")
        if (memo is None or memo[0] is not w or memo[1] is not a or memo[2] is not b or memo[3] is not bias
                or memo[4] is not packed):
            ok = (self._nf4_kernels_apply(torch.bfloat16) and _fused_ok(torch.empty(1, dtype=torch.bfloat16, device=w.device), w,
                                                                        self._adapter_rank())
                  and (bias is None or bias.dtype == torch.bfloat16))
            memo = (w, a, b, bias, packed, bool(ok))
            self.__dict__["_fused_memo"] = memo
        return memo[5] and x.is_cuda and x.numel() > 0

    def _base_out(self, x: torch.Tensor) -> torch.Tensor:
        """The frozen base layer by itself (composed path)."""
        if not self._quantize_base:
            return F.linear(x, self.weight, self.bias)
        out = linear_nf4(input=x, weight=self.weight)
        return out + self.bias if self.use_bias else out
