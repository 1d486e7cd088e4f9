"""``LoRALinear`` / ``QATLoRALinear`` with the QLoRA case running on fused HIP kernels.

Drop-in for ``torchtune.modules.peft.LoRALinear`` (``torchtune/modules/peft/lora.py:27-147``) and
``QATLoRALinear`` (``:150-306``): same constructor arguments, attributes (``in_dim, out_dim, rank, alpha,
use_bias, _quantize_base, disabled, merged, weight, bias, dropout, lora_a, lora_b``), parameter names,
initialisation and error messages.

With ``quantize_base=True``, bf16 activations on the GPU and a rank that is a multiple of 8, the whole layer

    y = x . D(W)^T (+ bias) + (alpha / rank) . (x . A^T) . B^T

is one autograd node: the adapter's hidden activation comes from a skinny MFMA kernel, everything else from
one GEMM that dequantises NF4 into LDS and folds the adapter in as extra contraction steps; the backward
mirrors it (``gx`` from one fused GEMM, ``gA``/``gB`` from two streaming reductions).  Only the packed weight,
``x`` and the [M, rank] hidden activation are kept for backward.  Other cases (fp32, odd ranks, other NF4
block sizes, adapter dropout in training) compose the same result from ``linear_nf4`` and ``F.linear``.
"""
from __future__ import annotations

from enum import Enum
from typing import List, Optional, Union

import torch
import torch.nn.functional as F
from torch import nn

from ... import ops
from ...nf4_tensor import _check_in_features, shape_and_dtype
from ._adapter_base import LowRankAdapterLinear, _lora_a_init_params, _lora_b_init_params  # noqa: F401


# One library call per direction of a QLoRA layer (False: the two stages of a direction are called one by one; same results)
ONE_CALL_PER_DIRECTION = True


class TrainableParams(Enum):
    FULL = "full"
    LORA = "lora"
    FROZEN = "frozen"


class _QLoRALinearFn(torch.autograd.Function):
    """Fused QLoRA linear.  Inputs: x [..., K] bf16, NF4 weight [N, K], lora_a [r, K], lora_b [N, r], bias or None.

    Each direction is one call into the library (``ttamd_qlora_linear_fwd_bf16`` / ``ttamd_qlora_linear_bwd_bf16``).  While a
    GEMM timer is installed (``ops.set_gemm_timer``) the two stages of a direction are called one by one instead - the
    same launches, the same bits - because the timer brackets the GEMM stage alone."""

    @staticmethod
    def forward(ctx, x, weight, lora_a, lora_b, bias, scale: float):
        N, K = shape_and_dtype(weight)[0]
        _check_in_features(x, weight)
        x2 = x.reshape(-1, K)
        tr = weight.backward_copy_for(x2.shape[0], True)
        # the expanded weight of a many-token call stays with the node when the backward will want a grad-input: its
        # GEMM then reads these tiles instead of expanding the weight again (ops.KEEP_FORWARD_TILES_MAX_TOKENS)
        # (only where that GEMM is the many-token launch: a grad-input of few output tiles stays on the fused kernel)
        keep = ctx.needs_input_grad[0] and ops.keeps_forward_tiles(x2.shape[0]) and ops.gemm_expands_weight(x2.shape[0], K, N)
        # expanded weights kept across calls (ops.RESIDENT_TILES_MAX_BYTES): a many-token forward runs on the tiles an
        # earlier one left with the weight, and leaves its own there when there are none yet
        resident = ops.resident_tiles_enabled() and ops.gemm_expands_weight(x2.shape[0], N, K)
        tiles = weight.resident_tiles() if resident else None
        if tiles is not None:
            h = ops.lora_hidden(x2, lora_a)
            y = ops.tiled_lora_linear(x2, tiles, N, h, lora_b, scale, True, bias, nf4_forward=True)
        elif ONE_CALL_PER_DIRECTION and not ops.gemm_timer_installed():
            y, h, tiles = ops.qlora_linear_fwd(x2, weight.quantized_data, weight.block_scalers(), N, lora_a, lora_b, scale, bias,
                                               block_scalers_t=tr[1] if tr else None, return_tiles=True)
            resident = resident and tiles is not None and weight.keep_resident_tiles(tiles)
        else:
            h = ops.lora_hidden(x2, lora_a)
            y, tiles = ops.nf4_lora_linear_fwd(x2, weight.quantized_data, weight.block_scalers(), N, h, lora_b, scale, bias,
                                               block_scalers_t=tr[1] if tr else None, return_tiles=True)
            resident = resident and tiles is not None and weight.keep_resident_tiles(tiles)
        if resident:  # the tiles exist anyway: the grad-input reads them wherever it is a many-token launch
            keep = ctx.needs_input_grad[0] and ops.gemm_expands_weight(x2.shape[0], K, N)
        # kept as a saved tensor, not as an attribute of the node: activation checkpointing then drops it with the other
        # saved tensors of the first pass and the recomputation brings it back, so that one layer's tiles are alive at a time
        ctx.save_for_backward(x2, h, weight, lora_a, lora_b, tiles if keep else None)
        ctx.scale = scale
        ctx.x_shape = x.shape
        ctx.has_bias = bias is not None
        return y.view(*x.shape[:-1], N)

    @staticmethod
    def backward(ctx, gy):
        x2, h, weight, lora_a, lora_b, kept = ctx.saved_tensors
        N, K = shape_and_dtype(weight)[0]
        gy2 = gy.reshape(-1, N)
        need_x, _, need_a, need_b, need_bias, _ = ctx.needs_input_grad
        gx = ga = gb = gbias = None
        if need_x or need_a or need_b:
            tiles = kept if need_x else None
            tr = weight.backward_copy_for(gy2.shape[0], False) if (need_x and tiles is None) else None
            if ONE_CALL_PER_DIRECTION and not ops.gemm_timer_installed():
                gx, ga, gb = ops.qlora_linear_bwd(gy2, x2, h, weight.quantized_data, weight.block_scalers(), lora_a, lora_b,
                                                  ctx.scale, transposed=tr, need_gx=need_x, tiles=tiles)
            else:
                gh, ga, gb = ops.lora_bwd(gy2, x2, h, lora_b, ctx.scale)
                if need_x and tiles is not None:
                    gx = ops.tiled_linear_dx(gy2, tiles, K, gh, lora_a, nf4_backward=True)
                elif need_x:
                    gx = ops.nf4_linear_bwd_dx(gy2, weight.quantized_data, weight.block_scalers(), K, gh, lora_a, transposed=tr)
            if need_x:
                gx = gx.view(ctx.x_shape)
            if not need_a:
                ga = None
            if not need_b:
                gb = None
        if ctx.has_bias and need_bias:
            gbias = gy2.sum(dim=0)
        return gx, None, ga, gb, gbias, None


class LoRALinear(LowRankAdapterLinear):
    """Linear layer with a low-rank adapter: ``x -> W0 x + (alpha / r) B A x``.

    Args:
        in_dim (int): input dimension
        out_dim (int): output dimension
        rank (int): rank of the adapter
        alpha (float): adapter scaling numerator
        dropout (float): dropout on the adapter's input. Default 0.0
        use_bias (bool): whether the base linear has a bias. Default False
        quantize_base (bool): hold the base weight as NF4. Default False
        **quantization_kwargs: forwarded to ``to_nf4`` (``block_size``, ``scaler_block_size``); only valid
            with ``quantize_base=True``

    Raises:
        ValueError: if quantisation arguments are given while ``quantize_base`` is False
    """

    def __init__(self, in_dim: int, out_dim: int, rank: int, alpha: float, dropout: float = 0.0, use_bias: bool = False,
                 quantize_base: bool = False, **quantization_kwargs):
        super().__init__()
        self.rank = rank
        self.alpha = alpha
        self._build(in_dim, out_dim, rank, dropout, use_bias, quantize_base, quantization_kwargs)
        self.merged = False
        self.initialize_parameters()

    def adapter_params(self) -> List[str]:
        """Names of this module's adapter parameters."""
        return ["lora_a.weight", "lora_b.weight"]

    def _fused(self, x: torch.Tensor) -> bool:
        return self._fused_path(x)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """x ``(..., in_dim)`` -> ``(..., out_dim)``"""
        scale = self.alpha / self.rank
        if not self.disabled and self._fused(x):
            return _QLoRALinearFn.apply(x, self.weight, self.lora_a.weight, self.lora_b.weight, self.bias, scale)
        out = self._base_out(x)
        if self.disabled:
            return out
        return out + scale * self.lora_b(self.lora_a(self.dropout(x)))


class _QATLoRATiledFn(torch.autograd.Function):
    """QAT + LoRA linear on the library's own GEMM.  Inputs: x [..., K] bf16 (the adapter's input), x_fq (the base path's
    input: x fake-quantised, or x itself), the frozen base weight's fake quantisation in the GEMM's tile order (forward
    and transposed), lora_a [r, K], lora_b [N, r].  The adapter product rides in the epilogue of the base GEMM in both
    directions; the activation's fake quantisation is straight-through, so the grad-input of both paths is one tensor."""

    @staticmethod
    def forward(ctx, x, x_fq, tiled_fwd, tiled_bwd, lora_a, lora_b, scale: float):
        N, K = lora_b.shape[0], lora_a.shape[1]
        x2 = x.reshape(-1, K)
        h = ops.lora_hidden(x2, lora_a)
        y = ops.tiled_lora_linear(x_fq.reshape(-1, K), tiled_fwd, N, h, lora_b, scale, lw_row_major=True)
        ctx.save_for_backward(x2, h, tiled_bwd, lora_a, lora_b)
        ctx.scale = scale
        ctx.x_shape = x.shape
        return y.view(*x.shape[:-1], N)

    @staticmethod
    def backward(ctx, gy):
        x2, h, tiled_bwd, lora_a, lora_b = ctx.saved_tensors
        N, K = lora_b.shape[0], lora_a.shape[1]
        gy2 = gy.reshape(-1, N)
        need_x, need_xfq, _, _, need_a, need_b, _ = ctx.needs_input_grad
        gh, ga, gb = ops.lora_bwd(gy2, x2, h, lora_b, ctx.scale)
        gx = None
        if need_x or need_xfq:
            gx = ops.tiled_lora_linear(gy2, tiled_bwd, K, gh, lora_a, 1.0, lw_row_major=False).view(ctx.x_shape)
        # x and x_fq are the same tensor up to the straight-through fake quantisation: the whole gradient goes to x
        return (gx if need_x else None), (gx if need_xfq and not need_x else None), None, None, ga if need_a else None, \
            gb if need_b else None, None


class QATLoRALinear(LoRALinear):
    """LoRA linear whose frozen base path sees fake-quantised activations and weights:
    ``x -> fq(W) fq(x) + (alpha / r) B A x``.

    Args:
        in_dim, out_dim, rank, alpha, dropout: as for :class:`LoRALinear`
        activation_qat_config (Optional[FakeQuantizeConfig]): how to fake-quantise the input; None = identity
        weight_qat_config (Optional[FakeQuantizeConfig]): how to fake-quantise the base weight; None = identity

    Raises:
        ValueError: if ``in_dim`` is not divisible by the weight ``group_size``
    """

    def __init__(
        self,
        in_dim: int,
        out_dim: int,
        rank: int,
        alpha: float,
        dropout: float = 0.0,
        activation_qat_config: Optional["FakeQuantizeConfig"] = None,  # noqa: F821
        weight_qat_config: Optional["FakeQuantizeConfig"] = None,  # noqa: F821
    ):
        super().__init__(in_dim, out_dim, rank, alpha, dropout, use_bias=False, quantize_base=False)
        from ...qat import FakeQuantizeConfig, FakeQuantizer

        if activation_qat_config is not None:
            assert isinstance(activation_qat_config, FakeQuantizeConfig)
            self.activation_fake_quantizer = FakeQuantizer(activation_qat_config)
        else:
            self.activation_fake_quantizer = nn.Identity()

        if weight_qat_config is not None:
            assert isinstance(weight_qat_config, FakeQuantizeConfig)
            group_size = weight_qat_config.group_size
            if group_size is not None and in_dim % group_size != 0:
                raise ValueError("in_dim (%s) must be divisible by group_size (%s)" % (in_dim, group_size))
            self.weight_fake_quantizer = FakeQuantizer(weight_qat_config)
        else:
            self.weight_fake_quantizer = nn.Identity()

    # The base weight of a QAT + LoRA layer is frozen, so its fake-quantised form only changes when the weight is
    # written (load_state_dict, copy_).  With 288 GB of HBM it is kept instead of being rebuilt in every forward; set
    # to False to recompute it each time, as the reference does.  A layer holds ONE form at a time: the row-major copy
    # (2 B per weight element; few-token calls) or the two tiled copies (forward and transposed, 4 B per element;
    # many-token calls), whichever its last call used - building one releases the other.  The cache key is the weight's
    # storage address, shape, dtype and version counter; a write through ``weight.data`` (``weight.data.copy_(...)``)
    # does not advance that counter, so code that writes this way calls ``invalidate_fake_quant_cache()`` afterwards.
    cache_frozen_weight_fake_quant = True

    def invalidate_fake_quant_cache(self) -> None:
        """Drop the kept fake-quantised forms of the frozen weight; the next forward rebuilds what it needs."""
        self._fq_weight_cache = None
        self._tiled_weight_cache = None

    def _fake_quantized_weight(self) -> torch.Tensor:
        w, fq = self.weight, self.weight_fake_quantizer
        cacheable = (
            self.cache_frozen_weight_fake_quant and not w.requires_grad and w.is_cuda and getattr(fq, "enabled", False)
        )
        if not cacheable:
            self._fq_weight_cache = None
            return fq(w)
        key = (w.data_ptr(), w._version, w.dtype, tuple(w.shape))
        cached = getattr(self, "_fq_weight_cache", None)
        if cached is None or cached[0] != key:
            with torch.no_grad():
                cached = (key, fq(w).detach())
            self._fq_weight_cache = cached
            self._tiled_weight_cache = None  # one form at a time
        return cached[1]

    # From this many tokens (and a full round of 256 x 256 output tiles in both directions) the layer runs on the library's
    # own GEMM: the frozen weight's fake quantisation is kept in the GEMM's tile order, forward and transposed (4 B per
    # element instead of the 2 B of the row-major copy), and the adapter product is part of the GEMM's epilogue.
    TILED_GEMM = True
    TILED_GEMM_MIN_ROWS = 2048

    def _tiled_weights(self):
        """(tiled_fwd, tiled_bwd) of the frozen weight's fake quantisation, rebuilt when the weight is written."""
        w, c = self.weight, self.weight_fake_quantizer.config
        key = (w.data_ptr(), w._version, tuple(w.shape), c.group_size, c.scale_precision, c.eps)
        cached = getattr(self, "_tiled_weight_cache", None)
        if cached is None or cached[0] != key:
            with torch.no_grad():
                tf, tb, scale = ops.fq_per_group_int4_sym_tiled(w.detach(), c.group_size, qparam_dtype=c.scale_precision, eps=c.eps)
            # what a call of the quantizer leaves behind
            self.weight_fake_quantizer.scale = scale.to(c.scale_precision)
            self.weight_fake_quantizer.zero_point = None
            cached = (key, tf, tb)
            self._tiled_weight_cache = cached
            self._fq_weight_cache = None  # one form at a time
        return cached[1], cached[2]

    def _tiled_ok(self, x: torch.Tensor) -> bool:
        from ...qat import FakeQuantizer, PerGroup

        q = self.weight_fake_quantizer
        if (not self.TILED_GEMM or self.disabled or not isinstance(q, FakeQuantizer) or not q.enabled or not x.is_cuda
                or x.dtype != torch.bfloat16 or self.weight.dtype != torch.bfloat16 or self.weight.requires_grad
                or self.lora_a.weight.dtype != torch.bfloat16 or self.rank % 8 != 0 or not 0 < self.rank <= 64
                or x.shape[-1] != self.in_dim or (self.training and getattr(self.dropout, "p", 0.0) > 0.0)):
            return False
        c = q.config
        if not (isinstance(c.granularity, PerGroup) and c.dtype == torch.int4 and c.is_symmetric):
            return False
        rows = x.numel() // self.in_dim
        full_round = ((rows + 255) // 256) * min(self.out_dim // 256, self.in_dim // 256) >= 256
        return rows >= self.TILED_GEMM_MIN_ROWS and full_round and ops.tiled_weight_shape_ok(self.out_dim, self.in_dim, c.group_size)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self._tiled_ok(x):
            tf, tb = self._tiled_weights()
            # the activation's fake quantisation is straight-through: its input takes the whole gradient inside the node
            return _QATLoRATiledFn.apply(x, self.activation_fake_quantizer(x).detach(), tf, tb, self.lora_a.weight,
                                         self.lora_b.weight, self.alpha / self.rank)
        out = F.linear(self.activation_fake_quantizer(x), self._fake_quantized_weight())
        if self.disabled:
            return out
        lora_out = self.lora_a(self.dropout(x))
        lora_out = (self.alpha / self.rank) * self.lora_b(lora_out)
        return out + lora_out

    @classmethod
    def from_lora_linear(
        cls,
        lora_linear: LoRALinear,
        activation_qat_config: Optional["FakeQuantizeConfig"] = None,  # noqa: F821
        weight_qat_config: Optional["FakeQuantizeConfig"] = None,  # noqa: F821
    ) -> "QATLoRALinear":
        """Build a ``QATLoRALinear`` that shares the weights and adapters of ``lora_linear``."""
        if lora_linear.bias is not None:
            raise ValueError("Bias is not supported in QAT + LoRA yet")
        if lora_linear._quantize_base:
            raise ValueError("quantize_base is not compatible with QAT + LoRA")
        p = lora_linear.dropout.p if isinstance(lora_linear.dropout, nn.Dropout) else 0.0
        new = cls(
            lora_linear.in_dim, lora_linear.out_dim, lora_linear.rank, lora_linear.alpha, p, activation_qat_config,
            weight_qat_config,
        )
        meta = torch.device("meta")
        # a meta-device source has no values to share (distributed construction)
        if lora_linear.weight.device != meta:
            new.weight = lora_linear.weight
        if lora_linear.lora_a.weight.device != meta:
            new.lora_a.weight = lora_linear.lora_a.weight
        if lora_linear.lora_b.weight.device != meta:
            new.lora_b.weight = lora_linear.lora_b.weight
        return new
