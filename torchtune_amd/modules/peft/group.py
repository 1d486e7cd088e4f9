"""LoRA linears that read the same input, computed as one group.

The reference calls such layers one after the other on one tensor: ``q_proj``, ``k_proj`` and ``v_proj`` in
``torchtune/modules/attention.py:234,262-263`` and ``w1`` / ``w3`` in ``torchtune/modules/feed_forward.py:50-53``, each a
``LoRALinear.forward`` (``torchtune/modules/peft/lora.py:128-147``).  ``lora_linear_group(x, layers)`` returns what those
calls return.  When every layer takes the fused QLoRA path it runs the group kernels instead: one pass over ``x`` for all
hidden activations ``x @ A_i.T``, one launch for the members' outputs at decode sizes, and in backward one pass over
``x`` for all ``grad A_i`` and a single grad-input GEMM over the members' concatenated output columns (fp32 sum over
the members, one rounding) in place of one GEMM per member plus the additions autograd would make.  Otherwise it
falls back to calling the layers in turn.
"""
from __future__ import annotations

from typing import List, Sequence, Tuple

import torch

from ... import nf4_tensor, ops
from ...nf4_tensor import _check_in_features
from .lora import LoRALinear


# The backward of ``silu(gate) * up`` inside the library call that multiplies its results with the pair's adapters (one pass
# over the two gradients less per layer at training sizes); False: ``ops.swiglu_bwd`` first.  Same results.
FUSED_SWIGLU_BWD = True


def _copies(weights, tokens: int):
    """The members' transposed copies for a call over ``tokens`` rows: none when the grouped grad-input runs on the
    expanded-weight path (it reads the weights' own codes), else every member's ``backward_copy()``."""
    if ops.group_dx_expands(tokens, weights[0].shape[1], [w.shape[0] for w in weights]):
        return [None] * len(weights)
    return [w.backward_copy() for w in weights]


class _QLoRAGroupFn(torch.autograd.Function):
    """Inputs: x [..., K], then per member (weight, lora_a, lora_b, bias or None); outputs: one y per member."""

    @staticmethod
    def forward(ctx, x, scales: Tuple[float, ...], *flat):
        n = len(scales)
        weights, las, lbs, biases = flat[0::4], flat[1::4], flat[2::4], flat[3::4]
        K = weights[0].shape[1]
        for w in weights:
            _check_in_features(x, w)
        x2 = x.reshape(-1, K)
        members = [ops.GroupMember(w.quantized_data, w.block_scalers(), tr, a, b, bias, s, w.shape[0])
                   for w, tr, a, b, bias, s in zip(weights, _copies(weights, x2.shape[0]), las, lbs, biases, scales)]
        h_cat, ys, kept = _group_forward(ctx, x2, members, weights, False)
        ctx.save_for_backward(x2, h_cat, *weights, *las, *lbs, kept)
        ctx.scales = scales
        ctx.x_shape = x.shape
        ctx.has_bias = tuple(b is not None for b in biases)
        outs = tuple(y.view(*x.shape[:-1], y.shape[-1]) for y in ys)
        return outs if n > 1 else outs[0]

    @staticmethod
    def backward(ctx, *gys):
        n = len(ctx.scales)
        saved = ctx.saved_tensors  # read once: activation checkpointing unpacks on every access
        x2, h_cat = saved[:2]
        rest, ctx.kept_tiles = saved[2:-1], saved[-1]
        weights, las, lbs = rest[:n], rest[n:2 * n], rest[2 * n:3 * n]
        gy2 = []
        for g, w in zip(gys, weights):
            # an output nobody used arrives as None
            gy2.append(torch.zeros(x2.shape[0], w.shape[0], dtype=x2.dtype, device=x2.device) if g is None
                       else g.reshape(-1, w.shape[0]))
        return _group_backward(ctx, x2, h_cat, weights, las, lbs, gy2)


def _group_forward(ctx, x2, members, weights, swiglu: bool):
    """``ops.lora_group_fwd`` on the expanded weights an earlier call left with the group where such tiles are kept across
    calls (``ops.RESIDENT_TILES_MAX_BYTES``), leaving this call's there when there are none yet; decides which tiles the
    node hands to its backward.  -> (h_cat, outputs, the tiles to save for backward or None)"""
    tokens = x2.shape[0]
    found = nf4_tensor.resident_group_tiles(weights, swiglu) if ops.resident_tiles_enabled() else None
    if found is not None:
        h_cat, outs, tiles, paired = ops.lora_group_fwd(x2, members, swiglu=swiglu, return_tiles=True, tiles=found[0], paired=found[1])
        resident = tiles is found[0]
    else:
        h_cat, outs, tiles, paired = ops.lora_group_fwd(x2, members, swiglu=swiglu, return_tiles=True)
        resident = (tiles is not None and ops.resident_tiles_enabled()
                    and nf4_tensor.keep_resident_group_tiles(weights, swiglu, tiles, paired))
    return h_cat, outs, _keep_tiles(ctx, tiles, paired, tokens, weights, resident)


def _keep_tiles(ctx, tiles, paired: bool, tokens: int, weights, resident: bool = False):
    """The group forward's expanded weights stay with the node when the backward will want a grad-input, the call is
    short enough for one expansion per layer to pay (``ops.KEEP_FORWARD_TILES_MAX_TOKENS``; any length when the tiles are
    kept across calls anyway) and the grouped grad-input is the many-token launch (with few output tiles it stays on the
    fused kernel).  Returns what the node saves for backward (the LAST of its saved tensors: a saved tensor, not an
    attribute of the node, so that activation checkpointing drops it with the first pass and the recomputation brings it
    back - one layer's tiles alive at a time), or None."""
    keep = (tiles is not None and ctx.needs_input_grad[0] and (resident or ops.keeps_forward_tiles(tokens))
            and ops.group_dx_expands(tokens, weights[0].shape[1], [w.shape[0] for w in weights]))
    ctx.tiles_paired = bool(keep and paired)
    return tiles if keep else None


def _group_backward(ctx, x2, h_cat, weights, las, lbs, gy2, swiglu=None):
    """Gradients of a group call in the order of its inputs (x, scales, then weight, lora_a, lora_b, bias per member).
    ``swiglu=(gact, gate, up)`` with ``gy2`` None: the output gradients are those of ``silu(gate) * up``, formed inside the
    library call (``ops.lora_group_bwd``); biases then get no gradient here (the gated pair has none)."""
    n = len(weights)
    need_x = ctx.needs_input_grad[0]
    tiles, paired = (ctx.kept_tiles, ctx.tiles_paired) if need_x else (None, False)
    ctx.kept_tiles = None
    copies = [None] * n if tiles is not None else _copies(weights, x2.shape[0])
    members = [ops.GroupMember(w.quantized_data, w.block_scalers(), tr, a, b, None, s, w.shape[0])
               for w, tr, a, b, s in zip(weights, copies, las, lbs, ctx.scales)]
    gx, grads, _ = ops.lora_group_bwd(x2, h_cat, members, gy2, want_gx=need_x, tiles=tiles, paired=paired, swiglu=swiglu)
    out: List = [gx.view(ctx.x_shape) if need_x else None, None]
    for i in range(n):
        _, need_a, need_b, need_bias = ctx.needs_input_grad[2 + 4 * i:6 + 4 * i]
        out += [None, grads[i][0] if need_a else None, grads[i][1] if need_b else None,
                gy2[i].sum(dim=0) if (gy2 is not None and ctx.has_bias[i] and need_bias) else None]
    return tuple(out)


class _QLoRAGatedFn(torch.autograd.Function):
    """``silu(w1(x)) * w3(x)`` for two LoRA linears over NF4 (``torchtune/modules/feed_forward.py:50-53``).  Inputs as
    for ``_QLoRAGroupFn`` with the members (w1, w3); the one output is the gated product.  The two projections are
    kept for backward, as autograd keeps them for the reference's separate multiply."""

    @staticmethod
    def forward(ctx, x, scales: Tuple[float, ...], *flat):
        weights, las, lbs, biases = flat[0::4], flat[1::4], flat[2::4], flat[3::4]
        K = weights[0].shape[1]
        for w in weights:
            _check_in_features(x, w)
        x2 = x.reshape(-1, K)
        members = [ops.GroupMember(w.quantized_data, w.block_scalers(), tr, a, b, bias, s, w.shape[0])
                   for w, tr, a, b, bias, s in zip(weights, _copies(weights, x2.shape[0]), las, lbs, biases, scales)]
        h_cat, (gate, up, act), kept = _group_forward(ctx, x2, members, weights, True)
        ctx.save_for_backward(x2, h_cat, gate, up, *weights, *las, *lbs, kept)
        ctx.scales = scales
        ctx.x_shape = x.shape
        ctx.has_bias = tuple(b is not None for b in biases)
        return act.view(*x.shape[:-1], act.shape[-1])

    @staticmethod
    def backward(ctx, gact):
        saved = ctx.saved_tensors
        x2, h_cat, gate, up = saved[:4]
        rest, ctx.kept_tiles = saved[4:-1], saved[-1]
        weights, las, lbs = rest[:2], rest[2:4], rest[4:6]
        if FUSED_SWIGLU_BWD and not any(ctx.has_bias):
            return _group_backward(ctx, x2, h_cat, weights, las, lbs, None, swiglu=(gact.reshape(gate.shape), gate, up))
        ggate, gup = ops.swiglu_bwd(gact.reshape(gate.shape), gate, up)
        return _group_backward(ctx, x2, h_cat, weights, las, lbs, [ggate, gup])


class _QLoRAFeedForwardFn(torch.autograd.Function):
    """``w2(silu(w1(x)) * w3(x))`` for three LoRA linears over NF4 (``torchtune/modules/feed_forward.py:50-53``).
    Inputs: x, the members' adapter scales, then (weight, lora_a, lora_b, bias or None) of w1, w3 and w2.  Forward as
    ``_QLoRAGatedFn`` followed by the fused linear; in backward the grad-input GEMM of w2 hands the gradients of the
    two projections straight to the pair's group backward: its result, the gradient of the gated product, meets gate
    and up in the GEMM's epilogue and is never written (``ops.nf4_linear_bwd_dx(..., swiglu=...)``)."""

    @staticmethod
    def forward(ctx, x, scales: Tuple[float, ...], *flat):
        weights, las, lbs, biases = flat[0::4], flat[1::4], flat[2::4], flat[3::4]
        K = weights[0].shape[1]
        for w in weights[:2]:
            _check_in_features(x, w)
        x2 = x.reshape(-1, K)
        members = [ops.GroupMember(w.quantized_data, w.block_scalers(), tr, a, b, bias, s, w.shape[0])
                   for w, tr, a, b, bias, s in zip(weights[:2], _copies(weights[:2], x2.shape[0]), las, lbs, biases, scales)]
        h_cat, (gate, up, act), kept = _group_forward(ctx, x2, members, weights[:2], True)
        w2 = weights[2]
        h2 = ops.lora_hidden(act, las[2])
        tr = w2.backward_copy_for(act.shape[0], True)
        y = ops.nf4_lora_linear_fwd(act, w2.quantized_data, w2.block_scalers(), w2.shape[0], h2, lbs[2], scales[2], biases[2],
                                    block_scalers_t=tr[1] if tr else None)
        ctx.save_for_backward(x2, h_cat, gate, up, act, h2, *weights, *las, *lbs, kept)
        ctx.scales = scales
        ctx.x_shape = x.shape
        ctx.has_bias = tuple(b is not None for b in biases)
        return y.view(*x.shape[:-1], y.shape[-1])

    @staticmethod
    def backward(ctx, gy):
        saved = ctx.saved_tensors
        x2, h_cat, gate, up, act, h2 = saved[:6]
        rest, ctx.kept_tiles = saved[6:-1], saved[-1]
        weights, las, lbs = rest[:3], rest[3:6], rest[6:9]
        w2 = weights[2]
        gy2 = gy.reshape(-1, w2.shape[0])
        gh2, ga2, gb2 = ops.lora_bwd(gy2, act, h2, lbs[2], ctx.scales[2])
        ggate, gup = ops.nf4_linear_bwd_dx(gy2, w2.quantized_data, w2.block_scalers(), w2.shape[1], gh2, las[2],
                                           transposed=w2.backward_copy_for(gy2.shape[0], False), swiglu=(gate, up))
        out = list(_group_backward(ctx, x2, h_cat, weights[:2], las[:2], lbs[:2], [ggate, gup]))
        _, need_a, need_b, need_bias = ctx.needs_input_grad[10:14]
        out += [None, ga2 if need_a else None, gb2 if need_b else None,
                gy2.sum(dim=0) if (ctx.has_bias[2] and need_bias) else None]
        return tuple(out)


def group_applies(x: torch.Tensor, layers: Sequence[torch.nn.Module]) -> bool:
    """True when ``lora_linear_group`` runs the group kernels for these layers on this input."""
    if not 1 <= len(layers) <= ops._lib.GROUP_MAX:
        return False
    for layer in layers:
        if type(layer) is not LoRALinear or layer.disabled or not layer._fused(x):
            return False
        if layer.in_dim != layers[0].in_dim:
            return False
    if not nf4_tensor.BACKWARD_COPY:
        # without the transposed copies the grouped grad-input exists only on the expanded-weight path (many tokens)
        M = x.numel() // layers[0].in_dim
        if not ops.group_dx_expands(M, layers[0].in_dim, [l.out_dim for l in layers]):
            return False
    return ops.group_shape_ok([l.out_dim for l in layers], layers[0].in_dim, [l.rank for l in layers])


def lora_swiglu_group(x: torch.Tensor, gate: torch.nn.Module, up: torch.nn.Module):
    """``silu(gate(x)) * up(x)`` (``torchtune/modules/feed_forward.py:50-53``) with the product formed in the epilogue of
    the pair's one GEMM launch where the group kernels apply; ``None`` when they do not (the caller multiplies itself)."""
    if not group_applies(x, (gate, up)) or gate.out_dim != up.out_dim:
        return None
    flat = []
    for layer in (gate, up):
        flat += [layer.weight, layer.lora_a.weight, layer.lora_b.weight, layer.bias]
    return _QLoRAGatedFn.apply(x, tuple(layer.alpha / layer.rank for layer in (gate, up)), *flat)


def lora_feed_forward(x: torch.Tensor, gate: torch.nn.Module, up: torch.nn.Module, down: torch.nn.Module):
    """``down(silu(gate(x)) * up(x))`` (``torchtune/modules/feed_forward.py:50-53``) as one autograd node: forward as
    ``lora_swiglu_group`` followed by ``down``; in backward ``down``'s grad-input GEMM writes the gradients of the two
    projections from its epilogue instead of the gradient of their product.  ``None`` when the group kernels do not
    apply to the pair or ``down`` does not take the fused path (the caller composes the layers itself)."""
    if not group_applies(x, (gate, up)) or gate.out_dim != up.out_dim:
        return None
    if type(down) is not LoRALinear or down.disabled or down.in_dim != gate.out_dim:
        return None
    probe = x.new_empty(1).expand(*x.shape[:-1], down.in_dim)  # x's device, dtype and token count; no memory
    if not down._fused(probe):
        return None
    flat = []
    for layer in (gate, up, down):
        flat += [layer.weight, layer.lora_a.weight, layer.lora_b.weight, layer.bias]
    return _QLoRAFeedForwardFn.apply(x, tuple(layer.alpha / layer.rank for layer in (gate, up, down)), *flat)


def lora_linear_group(x: torch.Tensor, layers: Sequence[torch.nn.Module]) -> Tuple[torch.Tensor, ...]:
    """``tuple(layer(x) for layer in layers)`` for layers that share the input ``x``."""
    if not group_applies(x, layers):
        return tuple(layer(x) for layer in layers)
    flat = []
    for layer in layers:
        flat += [layer.weight, layer.lora_a.weight, layer.lora_b.weight, layer.bias]
    out = _QLoRAGroupFn.apply(x, tuple(layer.alpha / layer.rank for layer in layers), *flat)
    return out if isinstance(out, tuple) else (out,)
