"""CPU oracle for the LoRA / QLoRA linear layer: forward and, through autograd, backward.

TEST INFRASTRUCTURE ONLY — never imported by the shipped package.

Restates ``LoRALinear.forward`` (``torchtune/modules/peft/lora.py:128-147``) op for op, with the reference's
rounding points: in bf16 each of ``linear_nf4``, ``lora_a``, ``lora_b``, the ``alpha/rank`` multiply and the
final add rounds to bf16.  The backward is whatever autograd derives from that graph, which is how the
reference obtains it (``LinearNF4.backward`` gives ``grad_out @ W.to(dtype)`` and no weight gradient).

Pinned by the reference's own known answers: mean(forward) == 1.1252 for the fixed-init layer of
``tests/torchtune/modules/peft/test_lora.py:111-116`` and 0.6291 without the bias (``:239-245``), by the
independent formula of ``tests/torchtune/models/llama2/scripts/compare_lora.py:99-112``, by closed forms for
the gradients and by ``torch.autograd.gradcheck`` in fp64 (tests/test_oracle_lora.py).
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

from . import nf4_oracle


class _LinearNF4(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, parts):
        ctx.parts = parts
        return nf4_oracle.linear_nf4_forward(x, parts)

    @staticmethod
    def backward(ctx, grad_out):
        return nf4_oracle.linear_nf4_backward(grad_out, ctx.parts), None


def lora_linear_forward(x, weight, lora_a, lora_b, alpha: float, rank: int, bias=None, disabled: bool = False):
    """`weight` is either a dense [N,K] tensor or an ``nf4_oracle.NF4Parts``."""
    if isinstance(weight, nf4_oracle.NF4Parts):
        out = _LinearNF4.apply(x, weight)
        if bias is not None:
            out = out + bias
    else:
        out = F.linear(x, weight, bias)
    if disabled:
        return out
    lora_out = F.linear(x, lora_a)
    lora_out = (alpha / rank) * F.linear(lora_out, lora_b)
    return out + lora_out


def lora_a_init_(a: torch.Tensor, generator=None) -> torch.Tensor:
    """kaiming-uniform with a = sqrt(5) (``torchtune/modules/peft/lora.py:309-313``): U(-1/sqrt(K), 1/sqrt(K))."""
    bound = 1.0 / math.sqrt(a.shape[1])
    with torch.no_grad():
        return a.uniform_(-bound, bound, generator=generator)


def fixed_init_tensor(shape, dtype=torch.float32) -> torch.Tensor:
    """arange(0, 1, 1/n).reshape(shape): the deterministic initialiser the reference's tests use
    (``tests/test_utils.py:206-225``)."""
    n = math.prod(shape)
    return torch.arange(0.0, 1.0, 1.0 / n, dtype=dtype).reshape(shape)


def merged_weight(parts: "nf4_oracle.NF4Parts", lora_a: torch.Tensor, lora_b: torch.Tensor, alpha: float, rank: int) -> torch.Tensor:
    """Checkpoint weight of a QLoRA linear: the state-dict hook's ``NF4Tensor.to(dtype)``
    (``torchtune/modules/common_utils.py:55-59``) followed by ``weight += (alpha / rank) * lora_b @ lora_a``
    (``torchtune/modules/peft/_utils.py:264-266``), eager ops in the weight dtype."""
    w = nf4_oracle.nf4_dequantize(parts).clone()
    w += (alpha / rank) * lora_b @ lora_a
    return w


def dora_linear_forward(x, weight, lora_a, lora_b, magnitude, alpha: float, rank: int, bias=None, disabled: bool = False):
    """``DoRALinear.forward`` (``torchtune/modules/peft/dora.py:156-192``) op for op.  ``weight`` is a dense tensor or
    the NF4 parts of one; the weight norm is a constant of the graph (``.detach()``, ``:183-184``)."""
    scaling = alpha / rank
    if isinstance(weight, nf4_oracle.NF4Parts):
        base_out = _LinearNF4.apply(x, weight)
        if bias is not None:
            base_out = base_out + bias
        dense = nf4_oracle.nf4_dequantize(weight).to(x.dtype)
    else:
        base_out = F.linear(x, weight, bias)
        dense = weight.to(x.dtype)
    if disabled:
        return base_out
    lora_out = F.linear(F.linear(x, lora_a), lora_b)
    x_eye = torch.eye(lora_a.shape[1], dtype=x.dtype)
    lora_weight = F.linear(F.linear(x_eye, lora_a), lora_b).T
    merged = dense + scaling * lora_weight.detach()
    weight_norm = torch.linalg.norm(merged, dim=1).to(merged.dtype).detach()
    mag_norm_scale = (magnitude / weight_norm).view(1, -1)
    dora_out = (mag_norm_scale - 1) * base_out + mag_norm_scale * lora_out * scaling
    return dora_out + base_out


def dora_weight_norm(weight, lora_a, lora_b, alpha: float, rank: int) -> torch.Tensor:
    """``DoRALinear._get_weight_norm`` as used by ``initialize_dora_magnitude`` (``dora.py:137-144``)."""
    dense = nf4_oracle.nf4_dequantize(weight).to(lora_a.dtype) if isinstance(weight, nf4_oracle.NF4Parts) else weight
    merged = dense + (alpha / rank) * (lora_b @ lora_a)
    return torch.linalg.norm(merged, dim=1).to(merged.dtype)
