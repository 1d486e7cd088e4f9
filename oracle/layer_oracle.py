"""CPU oracle for the memory-bound neighbours of the quantized linears: RMSNorm, rotary embedding, SwiGLU gate.

TEST INFRASTRUCTURE ONLY — never imported by the shipped package.

Eager-PyTorch restatements, op for op, of
* ``rms_norm``  <- ``RMSNorm.forward`` (``torchtune/modules/rms_norm.py:28-41``)
* ``rope_cache`` / ``rope`` <- ``Llama3ScaledRoPE`` without frequency scaling: the cache of ``build_rope_cache``
  (``torchtune/models/llama3_1/_position_embeddings.py:88-103``) and ``forward`` (``:128-190``, ``input_pos=None``)
* ``swiglu``    <- ``FeedForward.forward`` between the projections (``torchtune/modules/feed_forward.py:50-53``, ``nn.SiLU``)
Backward passes are whatever autograd derives from these graphs, as in the reference.

Pinned (tests/test_oracle_layer_ops.py) by the library routine ``torch.nn.functional.rms_norm`` in fp32, by closed
forms (unit-RMS output, constant rows), by the complex-multiplication form of the rotation and its invariants
(norm of every pair preserved, position 0 is the identity, inverse angle undoes it) and by ``F.silu`` in fp64.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def rms_norm(x: torch.Tensor, scale: torch.Tensor, eps: float) -> torch.Tensor:
    x_fp32 = x.float()
    x_normed = (x_fp32 * torch.rsqrt(x_fp32.pow(2).mean(-1, keepdim=True) + eps)).type_as(x)
    return x_normed * scale


def rope_cache(seq_len: int, head_dim: int, base: float) -> torch.Tensor:
    """[seq, head_dim/2, 2] fp32 table of (cos, sin)."""
    theta = 1.0 / (base ** (torch.arange(0, head_dim, 2)[: head_dim // 2].float() / head_dim))
    idx_theta = torch.einsum("i, j -> ij", torch.arange(seq_len, dtype=theta.dtype), theta).float()
    return torch.stack([torch.cos(idx_theta), torch.sin(idx_theta)], dim=-1)


def rope(x: torch.Tensor, cache: torch.Tensor) -> torch.Tensor:
    """x [b, s, n_h, h_d]"""
    seq_len = x.size(1)
    c = cache[:seq_len]
    xshaped = x.float().reshape(*x.shape[:-1], -1, 2)
    c = c.view(-1, xshaped.size(1), 1, xshaped.size(3), 2)
    x_out = torch.stack(
        [
            xshaped[..., 0] * c[..., 0] - xshaped[..., 1] * c[..., 1],
            xshaped[..., 1] * c[..., 0] + xshaped[..., 0] * c[..., 1],
        ],
        -1,
    )
    return x_out.flatten(3).type_as(x)


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    return F.silu(gate) * up


def cross_entropy_sum(logits: torch.Tensor, target: torch.Tensor, ignore_index: int = -100) -> torch.Tensor:
    """The per-chunk loss of ``LinearCrossEntropyLoss.compute_cross_entropy``
    (``torchtune/modules/loss/cross_entropy_loss.py:86-112``): the library routine itself."""
    return F.cross_entropy(logits.float(), target, reduction="sum", ignore_index=ignore_index)
