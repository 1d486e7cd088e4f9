"""RMSNorm, rotary embedding, the SwiGLU gate and the chunk cross entropy as single-pass HIP kernels with autograd.

These are the memory-bound neighbours of the quantized linears inside a decoder layer.  The reference runs each as
a chain of eager kernels: ``RMSNorm`` (``torchtune/modules/rms_norm.py:11-41``), ``Llama3ScaledRoPE.forward``
(``torchtune/models/llama3_1/_position_embeddings.py:128-190``), ``FeedForward.forward``
(``torchtune/modules/feed_forward.py:50-53``).  Same arguments and results (to floating-point tolerance); bf16
tensors on the GPU only, anything else raises.
"""
from __future__ import annotations

import torch
from torch import nn

from .. import ops


class _RMSNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, scale, eps: float):
        y, rstd = ops.rms_norm_fwd(x, scale, eps)
        ctx.save_for_backward(x, scale, rstd)
        return y.view(x.shape)

    @staticmethod
    def backward(ctx, gy):
        x, scale, rstd = ctx.saved_tensors
        gx, gscale = ops.rms_norm_bwd(gy, x, scale, rstd, want_gscale=ctx.needs_input_grad[1])
        return (gx.view(x.shape) if ctx.needs_input_grad[0] else None), gscale, None


class _AddRMSNormFn(torch.autograd.Function):
    """(x, residual, scale) -> (h = x + residual, RMSNorm(h)).  Backward: both inputs receive
    ``grad h + grad of the norm's input``, summed in the norm's backward pass."""

    @staticmethod
    def forward(ctx, x, residual, scale, eps: float):
        h, y, rstd = ops.add_rms_norm_fwd(x, residual, scale, eps)
        ctx.save_for_backward(h, scale, rstd)
        ctx.set_materialize_grads(False)  # an output nobody used arrives as None, not as a tensor of zeros
        return h.view(x.shape), y.view(x.shape)

    @staticmethod
    def backward(ctx, gh, gy):
        h, scale, rstd = ctx.saved_tensors
        if gy is None:  # the normalised output went nowhere
            return gh, gh, None, None
        gx, gscale = ops.rms_norm_bwd(gy, h, scale, rstd, want_gscale=ctx.needs_input_grad[2], g_add=gh)
        gx = gx.view(h.shape)
        return (gx if ctx.needs_input_grad[0] else None), (gx if ctx.needs_input_grad[1] else None), gscale, None


def add_rms_norm(x: torch.Tensor, residual: torch.Tensor, norm: "RMSNorm"):
    """``h = x + residual; return h, norm(h)``: the residual stream's addition and the norm of the next sub-block
    (``torchtune/modules/transformer.py:129-141``) as one pass forward and one backward; same bits as the separate ops."""
    return _AddRMSNormFn.apply(x, residual, norm.scale, norm.eps)


class RMSNorm(nn.Module):
    """Root-mean-square normalisation computed in fp32: ``bf16(x * rsqrt(mean(x^2) + eps)) * scale``.

    Args:
        dim (int): embedding size
        eps (float): added to the mean square. Default: 1e-6
    """

    def __init__(self, dim: int, eps: float = 1e-6) -> None:
        super().__init__()
        self.normalized_shape = (dim,)
        self.eps = eps
        self.scale = nn.Parameter(torch.ones(dim))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return _RMSNormFn.apply(x, self.scale, self.eps)


class _RopeFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, cache):
        ctx.save_for_backward(cache)
        return ops.rope(x, cache, inverse=False)

    @staticmethod
    def backward(ctx, gy):
        (cache,) = ctx.saved_tensors
        return ops.rope(gy, cache, inverse=True), None


def apply_rope(x: torch.Tensor, cache: torch.Tensor) -> torch.Tensor:
    """Rotate consecutive pairs of ``x [b, s, n_h, h_d]`` by the angles in ``cache [s, h_d/2, 2]`` (cos, sin), fp32 math."""
    return _RopeFn.apply(x, cache)


class _QKVRopeRepeatFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, cache):
        ctx.save_for_backward(cache)
        ctx.n_kv = k.shape[2]
        return ops.qkv_rope_repeat(q, k, v, cache)

    @staticmethod
    def backward(ctx, gq, gk, gv):
        (cache,) = ctx.saved_tensors
        return (*ops.qkv_rope_repeat_bwd(gq, gk, gv, cache, ctx.n_kv), None)


def qkv_rope_repeat(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cache: torch.Tensor):
    """What lies between the q / k / v projections and the attention (``torchtune/modules/attention.py:255-290``) as one
    kernel per direction: ``apply_rope(q)``, ``repeat_kv(apply_rope(k), rep)``, ``repeat_kv(v, rep)`` with
    ``rep = n_h // n_kv``, bit for bit."""
    return _QKVRopeRepeatFn.apply(q, k, v, cache)


class _RepeatKVFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, rep: int):
        ctx.rep = rep
        return ops.repeat_kv(x, rep)

    @staticmethod
    def backward(ctx, gy):
        return ops.repeat_kv_bwd(gy, ctx.rep), None


def repeat_kv(x: torch.Tensor, rep: int) -> torch.Tensor:
    """``x.unsqueeze(3).expand(b, s, n_kv, rep, h_d).flatten(2, 3)`` for ``x`` ``[b, s, n_kv, h_d]``: the grouped-query
    expansion of key / value heads (``torchtune/modules/attention.py:284-290``) as one copy kernel, with the sum over the
    copies as its backward."""
    return _RepeatKVFn.apply(x, rep)


class _SwiGLUFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, gate, up):
        ctx.save_for_backward(gate, up)
        return ops.swiglu_fwd(gate, up)

    @staticmethod
    def backward(ctx, gout):
        gate, up = ctx.saved_tensors
        gg, gu = ops.swiglu_bwd(gout, gate, up)
        return gg, gu


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``silu(gate) * up`` with the eager sequence's two bf16 roundings."""
    return _SwiGLUFn.apply(gate, up)


class _CrossEntropySumFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, target, ignore_index: int, scale: float):
        loss, grad = ops.cross_entropy_fwd_bwd(logits, target, ignore_index, scale)
        ctx.save_for_backward(grad)
        return loss.sum() * scale

    @staticmethod
    def backward(ctx, g):
        (grad,) = ctx.saved_tensors
        return grad.mul_(g.float().reshape(1)), None, None, None  # a 1-D fp32 factor: product in fp32, rounded to bf16 once


class _LinearCrossEntropySumFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, hidden, weight, target, ignore_index: int, scale: float):
        logits = torch.nn.functional.linear(hidden, weight)
        loss, grad = ops.cross_entropy_fwd_bwd(logits, target, ignore_index, scale)
        ctx.save_for_backward(grad, hidden, weight)
        return loss.sum() * scale

    @staticmethod
    def backward(ctx, g):
        grad, hidden, weight = ctx.saved_tensors
        gh = gw = None
        # the incoming scalar multiplies the small products, not the [rows, vocabulary] gradient of the logits
        if ctx.needs_input_grad[0]:
            gh = (grad @ weight).mul_(g.float().reshape(1))
        if ctx.needs_input_grad[1]:
            gw = (grad.t() @ hidden).mul_(g.float().reshape(1))
        return gh, gw, None, None, None


def linear_cross_entropy_sum(hidden: torch.Tensor, weight: torch.Tensor, target: torch.Tensor, ignore_index: int = -100,
                             scale: float = 1.0) -> torch.Tensor:
    """``scale * F.cross_entropy((hidden @ weight.T).float(), target, reduction="sum")`` for one chunk of rows: the
    vocabulary projection and the loss of the reference's ``LinearCrossEntropyLoss.compute_cross_entropy``
    (``torchtune/modules/loss/cross_entropy_loss.py:86-112``) as one autograd node, so that backward scales the
    ``[rows, dim]`` (and ``[vocabulary, dim]``) products by the incoming gradient instead of the logits' gradient."""
    return _LinearCrossEntropySumFn.apply(hidden, weight, target, ignore_index, scale)


def cross_entropy_sum(logits: torch.Tensor, target: torch.Tensor, ignore_index: int = -100, scale: float = 1.0) -> torch.Tensor:
    """``scale * F.cross_entropy(logits.float(), target, reduction="sum", ignore_index=ignore_index)`` for bf16 logits
    ``[rows, V]``: the per-chunk body of the reference's ``LinearCrossEntropyLoss``
    (``torchtune/modules/loss/cross_entropy_loss.py:86-112``).  The gradient w.r.t. the logits is produced in the same
    pass (pre-multiplied by ``scale``) and only rescaled by the incoming gradient in backward; call backward once."""
    return _CrossEntropySumFn.apply(logits, target, ignore_index, scale)
