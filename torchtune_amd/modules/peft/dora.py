"""``DoRALinear``: weight-decomposed low-rank adaptation, with the NF4 case on fused HIP kernels.

Drop-in for ``torchtune.modules.peft.DoRALinear`` (``torchtune/modules/peft/dora.py:21-192``): same constructor
arguments, attributes (``in_dim, out_dim, scaling, use_bias, _quantize_base, disabled, weight, bias, dropout,
lora_a, lora_b, magnitude``), methods (``to_empty, initialize_parameters, initialize_dora_magnitude,
adapter_params, forward``) and error messages.

    y = (m / ||W0 + s B A||_row) * (x W0^T + bias + s (x A^T) B^T),      s = alpha / rank

(the reference's ``(c - 1) base + c s lora + base`` with ``c = m / norm``).  With ``quantize_base=True``, bf16
activations on the GPU and a rank that is a multiple of 8, a forward is three launches: the row norms of the merged
weight straight from the packed codes (never materialising the [N, K] weight the reference builds twice per
call), the adapter's hidden activation, and the fused NF4 + LoRA GEMM with ``c`` applied per output column.  The
backward scales the incoming gradient by ``c`` and reduces the magnitude gradient in one pass, then runs the LoRA
backward.  Other cases compose the same result from ``linear_nf4`` / ``F.linear`` as the reference does.
"""
from __future__ import annotations

from typing import List, Optional, Union

import torch
from torch import nn

from ... import ops
from ...nf4_tensor import _check_in_features
from ._adapter_base import LowRankAdapterLinear


class _QDoRALinearFn(torch.autograd.Function):
    """Fused QDoRA linear: x [..., K] bf16, NF4 weight [N, K], lora_a [r, K], lora_b [N, r], magnitude [N], bias or None."""

    @staticmethod
    def forward(ctx, x, weight, lora_a, lora_b, magnitude, bias, scale: float):
        N, K = weight.shape
        _check_in_features(x, weight)
        x2 = x.reshape(-1, K)
        tr = weight.backward_copy_for(x2.shape[0], True)
        _, mns = ops.nf4_dora_weight_norm(weight.quantized_data, weight.block_scalers(), N, K, lora_a, lora_b, scale, magnitude)
        h = ops.lora_hidden(x2, lora_a)
        y = ops.nf4_lora_linear_fwd(x2, weight.quantized_data, weight.block_scalers(), N, h, lora_b, scale, bias,
                                    block_scalers_t=tr[1] if tr else None, col_scale=mns)
        ctx.save_for_backward(x2, h, y, mns, weight, lora_a, lora_b, magnitude)
        ctx.scale = scale
        ctx.x_shape = x.shape
        ctx.has_bias = bias is not None
        return y.view(*x.shape[:-1], N)

    @staticmethod
    def backward(ctx, gy):
        x2, h, y, mns, weight, lora_a, lora_b, magnitude = ctx.saved_tensors
        N, K = weight.shape
        need_x, _, need_a, need_b, need_m, need_bias, _ = ctx.needs_input_grad
        gy0, gmag = ops.dora_bwd_prologue(gy.reshape(-1, N), y, mns, magnitude)
        gx = ga = gb = gbias = None
        if need_x or need_a or need_b:
            gh, ga, gb = ops.lora_bwd(gy0, x2, h, lora_b, ctx.scale)
            if need_x:
                gx = ops.nf4_linear_bwd_dx(gy0, weight.quantized_data, weight.block_scalers(), K, gh, lora_a,
                                           transposed=weight.backward_copy_for(gy0.shape[0], False)).view(ctx.x_shape)
        if ctx.has_bias and need_bias:
            gbias = gy0.sum(dim=0)
        return gx, None, (ga if need_a else None), (gb if need_b else None), (gmag if need_m else None), gbias, None


class DoRALinear(LowRankAdapterLinear):
    """DoRA linear layer: ``x -> (m / ||W0 + (alpha / r) B A||) * (W0 x + (alpha / r) B A x)``.

    Args:
        in_dim (int): input dimension
        out_dim (int): output dimension
        rank (int): rank of the low-rank approximation
        alpha (float): scaling factor for the low-rank approximation
        dropout (float): dropout probability. Default: 0.0
        use_bias (bool): whether to include bias in the original linear layer. Default: False
        quantize_base (bool): hold the base weight as NF4. Default: False
        **quantization_kwargs: forwarded to ``to_nf4``; only valid with ``quantize_base=True``

    Raises:
        ValueError: If ``quantize_base`` is False, but quantization kwargs are provided.
    """

    def __init__(self, in_dim: int, out_dim: int, rank: int, alpha: float, dropout: float = 0.0, use_bias: bool = False,
                 quantize_base: bool = False, **quantization_kwargs):
        super().__init__()
        self.scaling = alpha / rank
        self._build(in_dim, out_dim, rank, dropout, use_bias, quantize_base, quantization_kwargs)
        self.magnitude = nn.Parameter(torch.empty(out_dim))
        self.initialize_parameters()

    def to_empty(self, *, device: Optional[Union[str, torch.device, int]], recurse: bool = True):
        super().to_empty(device=device, recurse=recurse)
        fresh = nn.Parameter(torch.empty_like(self.magnitude, device=device), requires_grad=self.magnitude.requires_grad)
        torch.utils.swap_tensors(self.magnitude, fresh)
        return self

    @torch.no_grad()
    def initialize_dora_magnitude(self):
        """Set the magnitude to the row norms of ``W0 + scaling * B A`` so that the layer starts out identical to LoRA.
        Call after the base and LoRA parameters are loaded.

        Raises:
            RuntimeError: If base or LoRA parameters are still on meta device.
        """
        if self.weight.is_meta or self.lora_a.weight.is_meta or self.lora_b.weight.is_meta:
            raise RuntimeError("Cannot initialize DoRA magnitude if base or LoRA parameters are still on meta device.")
        if self._nf4_kernels_apply(self.lora_a.weight.dtype):
            n, k = self.weight.shape
            norm, _ = ops.nf4_dora_weight_norm(self.weight.quantized_data, self.weight.block_scalers(), n, k,
                                               self.lora_a.weight, self.lora_b.weight, self.scaling)
        else:
            norm = self._get_weight_norm(self.weight.to(self.lora_a.weight.dtype), self.lora_b.weight @ self.lora_a.weight)
        self.magnitude.copy_(norm)

    def _get_weight_norm(self, weight, lora_weight):
        merged = weight + self.scaling * lora_weight
        return torch.linalg.norm(merged, dim=1).to(merged.dtype)

    def adapter_params(self) -> List[str]:
        """Names of this module's adapter parameters: ``lora_a.weight``, ``lora_b.weight`` and ``magnitude``."""
        return ["lora_a.weight", "lora_b.weight", "magnitude"]

    def _fused(self, x: torch.Tensor) -> bool:
        return self._fused_path(x) and self.magnitude.dtype == torch.bfloat16 and self.magnitude.is_cuda

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """x ``(..., in_dim)`` -> ``(..., out_dim)``"""
        if not self.disabled and self._fused(x):
            return _QDoRALinearFn.apply(x, self.weight, self.lora_a.weight, self.lora_b.weight, self.magnitude, self.bias,
                                        self.scaling)
        base_out = self._base_out(x)
        if self.disabled:
            return base_out
        # composed path, the reference's op order: the direction B A is read off an identity batch, its row norm is a
        # constant of the graph
        x = self.dropout(x)
        lora_out = self.lora_b(self.lora_a(x))
        eye = torch.eye(self.in_dim, device=self.lora_a.weight.device, dtype=x.dtype)
        direction = self.lora_b(self.lora_a(eye)).T.detach()
        norm = self._get_weight_norm(self.weight.to(x.dtype), direction).detach()
        c = (self.magnitude / norm).view(1, -1)
        return (c - 1) * base_out + c * lora_out * self.scaling + base_out
