"""Quantisation-aware training for the 8da4w scheme (int8 dynamic per-token activations, int4 per-group
symmetric weights) and the weight-only 4w scheme (uint4 per-group asymmetric weights with a floating-point zero
point) on the HIP fake-quant kernels.

The reference obtains all of this from ``torchao.quantization.qat``:

* ``Int8DynActInt4WeightQATQuantizer`` — re-exported at ``torchtune/training/quantization.py:26-29`` and
  instantiated from YAML by ``recipes/qat_single_device.py:375-386`` (``prepare``) and ``recipes/quantize.py:88-95``
  (``convert``);
* ``Int4WeightOnlyQATQuantizer`` — re-exported at ``torchtune/training/quantization.py:27`` and mapped to the
  ``"4w-qat"`` mode at ``:125-127``;
* ``FakeQuantizeConfig`` / ``FakeQuantizer`` — used directly by ``QATLoRALinear``
  (``torchtune/modules/peft/lora.py:222-250``);
* ``FakeQuantizedLinear`` — what ``_enable_linear_fake_quant`` toggles
  (``torchtune/training/quantization.py:56-71``).

The same names and call signatures are provided here.  Only the schemes named above have kernels;
any other configuration raises ``NotImplementedError`` instead of silently computing something else.
"""
from __future__ import annotations

from dataclasses import dataclass
from enum import Enum, auto
import threading
import weakref
from typing import Optional, Tuple, Union

import torch
import torch.nn.functional as F
from torch import nn

from . import ops


@dataclass
class PerToken:
    """One set of qparams per row of the last dimension."""


@dataclass
class PerGroup:
    """One set of qparams per ``group_size`` consecutive elements of the last dimension."""

    group_size: int


class ZeroPointDomain(Enum):
    """Whether the zero point lives on the integer grid or in the floating-point domain."""

    INT = auto()
    FLOAT = auto()
    NONE = auto()


class FakeQuantizeConfig:
    """How a tensor is fake-quantised.

    Args:
        dtype: ``torch.int8`` (activations), ``torch.int4`` (weights) or ``torch.uint4`` (weight-only scheme)
        granularity: ``"per_token"``, ``"per_group"``, a ``PerToken()`` or a ``PerGroup(n)``
        group_size: keyword shortcut for ``PerGroup(group_size)``
        is_symmetric: symmetric (zero-point 0) or asymmetric mapping
        scale_precision, zero_point_precision: dtypes of the qparams kept on the quantizer
        is_dynamic: qparams are recomputed from each input (the only supported mode)
        zero_point_domain: ``ZeroPointDomain.INT`` (default) or ``ZeroPointDomain.FLOAT`` (the weight-only scheme)
        eps: lower bound of the scale; None keeps the scheme's default
    """

    def __init__(
        self,
        dtype: torch.dtype,
        granularity: Union[str, PerToken, PerGroup, None] = None,
        mapping_type: Optional[str] = None,
        scale_precision: torch.dtype = torch.float32,
        zero_point_precision: torch.dtype = torch.int32,
        is_dynamic: bool = True,
        *,
        group_size: Optional[int] = None,
        is_symmetric: Optional[bool] = None,
        zero_point_domain: ZeroPointDomain = ZeroPointDomain.INT,
        eps: Optional[float] = None,
    ):
        if dtype not in (torch.int8, torch.int4, torch.uint4):
            raise NotImplementedError(f"FakeQuantizeConfig: dtype {dtype} has no kernel (int8, int4 and uint4 do)")
        self.dtype = dtype
        if zero_point_domain not in (ZeroPointDomain.INT, ZeroPointDomain.FLOAT):
            raise ValueError("Please use ZeroPointDomain.INT or ZeroPointDomain.FLOAT")
        self.zero_point_domain = zero_point_domain
        if group_size is not None and granularity is not None and granularity != "per_group":
            raise ValueError("`group_size` conflicts with granularity '%s'" % (granularity,))
        if isinstance(granularity, str):
            if granularity == "per_token":
                granularity = PerToken()
            elif granularity == "per_group":
                if group_size is None:
                    raise ValueError("Granularity was 'per_group' but no `group_size` was set")
                granularity = PerGroup(group_size)
            else:
                raise ValueError(f"Unexpected granularity: '{granularity}'; expected 'per_token' or 'per_group'")
        elif granularity is None:
            if group_size is None:
                raise ValueError("At least one of `granularity` or `group_size` must be set")
            granularity = PerGroup(group_size)
        if not isinstance(granularity, (PerToken, PerGroup)):
            raise ValueError(f"Granularity '{granularity}' is not supported")
        self.granularity = granularity
        if mapping_type is not None and is_symmetric is not None:
            raise ValueError("Cannot set both `mapping_type` and `is_symmetric`")
        if mapping_type is not None:
            if str(mapping_type).lower().endswith("asymmetric"):
                is_symmetric = False
            elif str(mapping_type).lower().endswith("symmetric"):
                is_symmetric = True
            else:
                raise ValueError(f"Unexpected mapping_type: {mapping_type}")
        self.is_symmetric = True if is_symmetric is None else bool(is_symmetric)
        self.scale_precision = scale_precision
        self.zero_point_precision = zero_point_precision
        self.is_dynamic = is_dynamic
        # lower bound of the scale; None = the scheme's default (finfo(float32).eps for the integer schemes, 1e-6 for
        # the weight-only uint4 scheme).  Versions of the reference's quantisation package differ here.
        self.eps = eps
        if not is_dynamic:
            raise NotImplementedError("FakeQuantizeConfig: only dynamic qparams have a kernel")

    @property
    def group_size(self) -> Optional[int]:
        return self.granularity.group_size if isinstance(self.granularity, PerGroup) else None

    @property
    def mapping_type(self) -> str:
        return "SYMMETRIC" if self.is_symmetric else "ASYMMETRIC"

    def __repr__(self) -> str:
        return (
            f"FakeQuantizeConfig(dtype={self.dtype}, granularity={self.granularity}, mapping_type={self.mapping_type}, "
            f"scale_precision={self.scale_precision}, zero_point_precision={self.zero_point_precision}, "
            f"is_dynamic={self.is_dynamic})"
        )


class _StraightThrough(torch.autograd.Function):
    """y = fake_quantise(x); dy/dx = 1.  The reference masks the gradient with (qmin <= q <= qmax) evaluated on the
    already clamped q, which is identically true."""

    @staticmethod
    def forward(ctx, x, fq):
        return fq

    @staticmethod
    def backward(ctx, g):
        return g, None


class FakeQuantizer(nn.Module):
    """Fake-quantise the input according to ``config``.  ``enabled = False`` makes it the identity."""

    def __init__(self, config: FakeQuantizeConfig):
        super().__init__()
        self.config = config
        self.enabled = True
        self.scale: Optional[torch.Tensor] = None
        self.zero_point: Optional[torch.Tensor] = None
        g = config.granularity
        if config.scale_precision not in (torch.float32, torch.bfloat16):
            raise NotImplementedError("fake quantisation has kernels for float32 and bfloat16 scale_precision only")
        if isinstance(g, PerToken):
            if config.dtype != torch.int8 or config.is_symmetric:
                raise NotImplementedError("per-token fake quantisation has a kernel for asymmetric int8 only")
        elif isinstance(g, PerGroup):
            sym_int4 = config.dtype == torch.int4 and config.is_symmetric and config.zero_point_domain == ZeroPointDomain.INT
            if not (sym_int4 or self._weight_only_int4(config)):
                raise NotImplementedError(
                    "per-group fake quantisation has kernels for symmetric int4 and for asymmetric uint4 with a "
                    "floating-point zero point only")

    @staticmethod
    def _weight_only_int4(config: FakeQuantizeConfig) -> bool:
        return (config.dtype == torch.uint4 and not config.is_symmetric and config.zero_point_domain == ZeroPointDomain.FLOAT
                and config.scale_precision in (torch.bfloat16, torch.float32)
                and config.zero_point_precision == config.scale_precision)

    # Sibling linears (q/k/v, gate/up) fake-quantise the very same activation tensor one after the other; the dynamic
    # per-token result depends on the tensor and the scale precision only, so the last one is kept (per thread, with a
    # weak reference to the tensor: the entry is dropped when the tensor dies, so its address cannot come back as another
    # tensor's) and reused while the same, unmodified tensor object comes in again.
    # ``share_identical_inputs = False`` recomputes every time.
    share_identical_inputs = True
    _last = threading.local()

    def _per_token(self, x: torch.Tensor):
        # Inference tensors keep no version counter (reading it raises), so nothing is shared under inference_mode.
        share = FakeQuantizer.share_identical_inputs and not (torch.is_inference_mode_enabled() or x.is_inference())
        if not share:
            FakeQuantizer._last.entry = None
            return ops.fq_per_token_int8_asym(x.detach(), qparam_dtype=self.config.scale_precision, eps=self.config.eps)
        key = (x._version, self.config.scale_precision, self.config.eps)
        hit = getattr(FakeQuantizer._last, "entry", None)
        if hit is not None and hit[0]() is x and hit[1] == key:
            return hit[2]
        out = ops.fq_per_token_int8_asym(x.detach(), qparam_dtype=self.config.scale_precision, eps=self.config.eps)
        # the input is held by weak reference: the entry dies with the activation instead of keeping it (and its
        # fake-quantised copy) alive after the step; a new tensor replaces the entry
        try:
            FakeQuantizer._last.entry = (weakref.ref(x, FakeQuantizer._drop_entry), key, out)
        except TypeError:
            FakeQuantizer._last.entry = None
        return out

    @staticmethod
    def forget_shared_input() -> None:
        """Drop the calling thread's kept per-token result (it holds a fake-quantised copy of one activation)."""
        FakeQuantizer._last.entry = None

    @staticmethod
    def _drop_entry(_ref) -> None:
        hit = getattr(FakeQuantizer._last, "entry", None)
        if hit is not None and hit[0] is _ref:
            FakeQuantizer._last.entry = None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if not self.enabled:
            return x
        with torch.no_grad():
            if isinstance(self.config.granularity, PerToken):
                fq, scale, zp = self._per_token(x)
                self.scale = scale.to(self.config.scale_precision)
                self.zero_point = zp.to(self.config.zero_point_precision)
            else:
                gs = self.config.group_size
                if x.shape[-1] % gs != 0:
                    raise ValueError(f"last dimension ({x.shape[-1]}) must be divisible by group_size ({gs})")
                if self._weight_only_int4(self.config):
                    fq, scale, zp = ops.fq_per_group_uint4_asym(x.detach(), gs, self.config.scale_precision, min_scale=self.config.eps)
                    self.scale = scale.to(self.config.scale_precision)
                    self.zero_point = zp.to(self.config.zero_point_precision)
                else:
                    fq, scale = ops.fq_per_group_int4_sym(x.detach(), gs, qparam_dtype=self.config.scale_precision, eps=self.config.eps)
                    self.scale = scale.to(self.config.scale_precision)
                    self.zero_point = None
        return _StraightThrough.apply(x, fq.view(x.shape))

    def __repr__(self) -> str:
        return f"FakeQuantizer({self.config})"


# FakeQuantizedLinear on the library's own GEMM: the weight's fake quantisation is written in the GEMM's tile order (once
# for the forward, once transposed for the grad-input) and never row-major; forward and grad-input run on
# ``ttamd_tiled_linear_bf16``, the weight gradient on ``ttamd_gemm_tn_bf16`` (layers of fewer than 192 output tiles of
# 256 x 256: the vendor library).  Taken from ``TILED_GEMM_MIN_ROWS`` tokens and a full round of 256 x 256 tiles on the
# 256 CUs in both directions (``TILED_GEMM_MIN_TILES``); with fewer, the vendor library's smaller tiles fill the chip
# better (M = 2048, 4096 x 4096: 62 against 80 us).  ``TILED_GEMM = False``: row-major fq(W) and ``F.linear`` for everything.
TILED_GEMM = True
TILED_GEMM_MIN_ROWS = 2048
TILED_GEMM_MIN_TILES = 256
TN_GEMM_MIN_TILES = 192
# the weight gradients of a group's members (they share fq(x)) as one launch; False: one launch per member (A/B timing)
TN_GROUP_GEMM = True


class _TiledFakeQuantLinearFn(torch.autograd.Function):
    """y = x @ fq(W).T + b with fq = per-group symmetric int4 fake quantisation (straight-through for W).  ``x`` arrives
    already fake-quantised (or not) by the activation quantizer."""

    @staticmethod
    def forward(ctx, x, weight, bias, quantizer):
        c = quantizer.config
        N, K = weight.shape
        x2 = x.reshape(-1, K)
        need_gx = ctx.needs_input_grad[0]
        tf, tb, scale = ops.fq_per_group_int4_sym_tiled(weight.detach(), c.group_size, forward=True, backward=need_gx,
                                                        qparam_dtype=c.scale_precision, eps=c.eps)
        quantizer.scale = scale.to(c.scale_precision)
        quantizer.zero_point = None
        y = ops.tiled_linear(x2, tf, N, bias)
        ctx.save_for_backward(x2, tb)
        ctx.x_shape = x.shape
        ctx.shape = (N, K)
        ctx.has_bias = bias is not None
        return y.view(*x.shape[:-1], N)

    @staticmethod
    def backward(ctx, gy):
        x2, tb = ctx.saved_tensors
        N, K = ctx.shape
        gy2 = gy.reshape(-1, N)
        need_x, need_w, need_b, _ = ctx.needs_input_grad
        gx = ops.tiled_linear(gy2, tb, K).view(ctx.x_shape) if need_x else None
        gw = None
        if need_w:
            # a few hundred output tiles fill the chip: the transposing GEMM of this library (1.2 - 1.3 PFLOP/s at the 8B
            # shapes against 0.95 - 1.1 for the vendor library's); narrower layers (k / v) stay on the vendor library
            own = ops.gemm_tn_applies(gy2.shape[0], N, K) and (N // 256) * (K // 256) >= TN_GEMM_MIN_TILES
            gw = ops.gemm_tn(gy2, x2) if own else gy2.t().matmul(x2)
        gb = gy2.sum(dim=0) if (ctx.has_bias and need_b) else None
        return gx, gw, gb, None


class _TiledFakeQuantLinearCrossEntropySumFn(torch.autograd.Function):
    """``scale * cross_entropy(x @ fq(W).T, target, reduction="sum")`` as one node: the vocabulary projection of a
    fake-quantised output layer and the loss of one chunk of rows (the reference: ``LinearCrossEntropyLoss.compute_cross_entropy``,
    ``torchtune/modules/loss/cross_entropy_loss.py:86-112``, on a ``FakeQuantizedLinear``).  The loss kernel leaves the
    gradient of the logits; in backward the incoming scalar multiplies the ``[rows, dim]`` operands of the two products
    instead of that ``[rows, vocabulary]`` gradient (1 GB per chunk at 4096 x 128256)."""

    @staticmethod
    def forward(ctx, x, weight, quantizer, target, ignore_index: int, scale: float):
        c = quantizer.config
        N, K = weight.shape
        x2 = x.reshape(-1, K)
        need_gx = ctx.needs_input_grad[0]
        tf, tb, qscale = ops.fq_per_group_int4_sym_tiled(weight.detach(), c.group_size, forward=True, backward=need_gx,
                                                         qparam_dtype=c.scale_precision, eps=c.eps)
        quantizer.scale = qscale.to(c.scale_precision)
        quantizer.zero_point = None
        logits = ops.tiled_linear(x2, tf, N)
        loss, grad = ops.cross_entropy_fwd_bwd(logits, target.reshape(-1), ignore_index, scale)
        ctx.save_for_backward(grad, x2, tb)
        ctx.x_shape = x.shape
        ctx.shape = (N, K)
        return loss.sum() * scale

    @staticmethod
    def backward(ctx, g):
        grad, x2, tb = ctx.saved_tensors
        N, K = ctx.shape
        need_x, need_w = ctx.needs_input_grad[:2]
        g1 = g.float().reshape(1)  # a 1-D fp32 factor: products in fp32, rounded to bf16 once
        gx = ops.tiled_linear(grad, tb, K).mul_(g1).view(ctx.x_shape) if need_x else None
        gw = None
        if need_w:
            xs = x2.clone().mul_(g1)
            own = ops.gemm_tn_applies(grad.shape[0], N, K) and (N // 256) * (K // 256) >= TN_GEMM_MIN_TILES
            gw = ops.gemm_tn(grad, xs) if own else grad.t().matmul(xs)
        return gx, gw, None, None, None, None


class _TiledFakeQuantGroupFn(torch.autograd.Function):
    """Fake-quantised linears that read the same (already fake-quantised) input, as one node: every weight's fake
    quantisation goes into one stack of tiles per direction, the forward is one GEMM launch over the members' output
    columns, the grad-input one launch over their concatenated contraction (fp32 sum over the members, one rounding, no
    additions of partial grad-inputs afterwards).  Inputs: x, then per member (weight, bias or None); ``quantizers`` are
    the members' weight quantizers (same config)."""

    @staticmethod
    def forward(ctx, x, quantizers, swiglu: bool, *flat):
        weights, biases = flat[0::2], flat[1::2]
        c = quantizers[0].config
        K = weights[0].shape[1]
        x2 = x.reshape(-1, K)
        need_gx = ctx.needs_input_grad[0]
        tf, tb, scales = ops.fq_int4_sym_tiled_group([w.detach() for w in weights], c.group_size, forward=True, backward=need_gx,
                                                     qparam_dtype=c.scale_precision, eps=c.eps, paired=swiglu)
        for q, s in zip(quantizers, scales):
            q.scale = s.to(c.scale_precision)
            q.zero_point = None
        ys = ops.tiled_linear_group_fwd(x2, tf, [w.shape[0] for w in weights], biases, swiglu=swiglu)
        ctx.x_shape = x.shape
        ctx.shapes = tuple(tuple(w.shape) for w in weights)
        ctx.has_bias = tuple(b is not None for b in biases)
        ctx.swiglu = swiglu
        if swiglu:  # ``silu(w1 x) * w3 x`` (torchtune/modules/feed_forward.py:50-53) from the launch's epilogue: the one output
            ctx.save_for_backward(x2, tb, ys[0], ys[1])
            return ys[2].view(*x.shape[:-1], ys[2].shape[-1])
        ctx.save_for_backward(x2, tb)
        return tuple(y.view(*x.shape[:-1], y.shape[-1]) for y in ys)

    @staticmethod
    def backward(ctx, *gys):
        if ctx.swiglu:
            x2, tb, gate, up = ctx.saved_tensors
            gys = ops.swiglu_bwd(gys[0].reshape(gate.shape), gate, up)
        else:
            x2, tb = ctx.saved_tensors
        K = ctx.shapes[0][1]
        gy2 = [torch.zeros(x2.shape[0], N, dtype=x2.dtype, device=x2.device) if g is None else g.reshape(-1, N)
               for g, (N, _) in zip(gys, ctx.shapes)]
        out = [ops.tiled_linear_group_dx(gy2, tb, K).view(ctx.x_shape) if ctx.needs_input_grad[0] else None, None, None]
        # the members' weight gradients share fq(x): one launch over their stacked rows when every member wants one (a
        # narrow member then fills the rounds of the wide ones instead of a launch of its own on the vendor library)
        M = x2.shape[0]
        need_ws = [ctx.needs_input_grad[3 + 2 * i] for i in range(len(ctx.shapes))]
        gws = None
        if (TN_GROUP_GEMM and len(ctx.shapes) > 1 and all(need_ws) and all(ops.gemm_tn_applies(M, N, K) for N, _ in ctx.shapes)
                and sum(N // 256 for N, _ in ctx.shapes) * (K // 256) >= TN_GEMM_MIN_TILES):
            gws = ops.gemm_tn_group(gy2, x2)
        for i, (N, _) in enumerate(ctx.shapes):
            need_w, need_b = ctx.needs_input_grad[3 + 2 * i:5 + 2 * i]
            gw = None
            if gws is not None:
                gw = gws[i]
            elif need_w:
                own = ops.gemm_tn_applies(M, N, K) and (N // 256) * (K // 256) >= TN_GEMM_MIN_TILES
                gw = ops.gemm_tn(gy2[i], x2) if own else gy2[i].t().matmul(x2)
            out += [gw, gy2[i].sum(dim=0) if (ctx.has_bias[i] and need_b) else None]
        return tuple(out)


def fake_quantized_swiglu_group(x: torch.Tensor, gate, up) -> Optional[torch.Tensor]:
    """``silu(gate(x)) * up(x)`` (``torchtune/modules/feed_forward.py:50-53``) for two ``FakeQuantizedLinear`` layers, with the
    product written by the pair's one GEMM launch; ``None`` where the group kernels do not apply (the caller multiplies)."""
    if not _group_tiled_ok(x, (gate, up)) or gate.out_features != up.out_features:
        return None
    return fake_quantized_linear_group(x, (gate, up), swiglu=True)


def fake_quantized_linear_group(x: torch.Tensor, layers, swiglu: bool = False) -> Tuple[torch.Tensor, ...]:
    """``tuple(layer(x) for layer in layers)`` for ``FakeQuantizedLinear`` layers that read the same input (``q_proj`` /
    ``k_proj`` / ``v_proj``, ``torchtune/modules/attention.py:234,262-263``; ``w1`` / ``w3``,
    ``torchtune/modules/feed_forward.py:50-53``).  When every member is the 8da4w kind with one configuration and the
    shapes give the library's GEMM full rounds of tiles, the group runs as one node (``_TiledFakeQuantGroupFn``): narrow
    members (the 1024-wide k / v projections) ride in the wide launch instead of falling back to the vendor library, and
    the members' grad-inputs are summed inside the GEMM.  Otherwise the layers are called in turn."""
    if not _group_tiled_ok(x, layers):
        if swiglu:
            raise ValueError("fake_quantized_linear_group: the gated product needs a pair the group kernels serve")
        return tuple(layer(x) for layer in layers)
    first = layers[0]
    a0 = first.activation_fake_quantizer
    xq = x if a0 is None else a0(x)
    # every member's quantizer ends up with the qparams a call of its own would have recorded: the members' activation
    # configurations are equal (_group_tiled_ok), so the first member's are theirs and no kernel runs again
    if a0 is not None and a0.enabled:
        for layer in layers[1:]:
            layer.activation_fake_quantizer.scale = a0.scale
            layer.activation_fake_quantizer.zero_point = a0.zero_point
        FakeQuantizer.forget_shared_input()  # the group was the shared result's last user: do not keep fq(x) alive
    flat = []
    for layer in layers:
        flat += [layer.weight, layer.bias]
    out = _TiledFakeQuantGroupFn.apply(xq, tuple(layer.weight_fake_quantizer for layer in layers), swiglu, *flat)
    return out


def _group_tiled_ok(x: torch.Tensor, layers) -> bool:
    if not TILED_GEMM or not 2 <= len(layers) <= ops._lib.GROUP_MAX or not x.is_cuda or x.dtype != torch.bfloat16:
        return False
    first = layers[0]
    for layer in layers:
        q = getattr(layer, "weight_fake_quantizer", None)
        if (not isinstance(layer, FakeQuantizedLinear) or q is None or not q.enabled or layer.weight.dtype != torch.bfloat16
                or layer.in_features != first.in_features or layer.out_features % 256 != 0):
            return False
        c, c0 = q.config, first.weight_fake_quantizer.config
        if not (isinstance(c.granularity, PerGroup) and c.dtype == torch.int4 and c.is_symmetric and c.group_size == c0.group_size
                and c.scale_precision == c0.scale_precision and c.eps == c0.eps):
            return False
        a, a0 = layer.activation_fake_quantizer, first.activation_fake_quantizer
        if (a is None) != (a0 is None) or (a is not None and (a.enabled != a0.enabled or repr(a.config) != repr(a0.config))):
            return False
    K = first.in_features
    rows = x.numel() // max(1, x.shape[-1])
    n_total = sum(layer.out_features for layer in layers)
    row_tiles = (rows + 255) // 256
    return (x.shape[-1] == K and rows >= TILED_GEMM_MIN_ROWS and row_tiles * min(n_total // 256, K // 256) >= TILED_GEMM_MIN_TILES
            and ops.tiled_weight_shape_ok(n_total, K, first.weight_fake_quantizer.config.group_size))


class FakeQuantizedLinear(nn.Linear):
    """``nn.Linear`` that fake-quantises its input and/or weight before the matmul."""

    def __init__(
        self,
        in_features: int,
        out_features: int,
        bias: bool = False,
        activation_config: Optional[FakeQuantizeConfig] = None,
        weight_config: Optional[FakeQuantizeConfig] = None,
        *args,
        **kwargs,
    ) -> None:
        super().__init__(in_features, out_features, bias, *args, **kwargs)
        self.activation_fake_quantizer = FakeQuantizer(activation_config) if activation_config is not None else None
        if weight_config is not None:
            gs = weight_config.group_size
            if gs is not None and in_features % gs != 0:
                raise ValueError("in_features (%s) %% group_size (%s) must be == 0" % (in_features, gs))
            self.weight_fake_quantizer = FakeQuantizer(weight_config)
        else:
            self.weight_fake_quantizer = None

    def _tiled_ok(self, x: torch.Tensor) -> bool:
        """The weight is fake-quantised straight into the layout of the library's own GEMM (no row-major fq(W), forward
        and grad-input on ``ttamd_tiled_linear_bf16``) when ``TILED_GEMM`` is set and the layer is the 8da4w kind: bf16,
        per-group symmetric int4 weight, shapes the kernels serve, a few thousand tokens."""
        q = self.weight_fake_quantizer
        if not TILED_GEMM or q is None or not q.enabled or not x.is_cuda or x.dtype != torch.bfloat16 or self.weight.dtype != torch.bfloat16:
            return False
        c = q.config
        if not (isinstance(c.granularity, PerGroup) and c.dtype == torch.int4 and c.is_symmetric):
            return False
        rows = x.numel() // max(1, x.shape[-1])
        # a full round of 256 x 256 output tiles on the 256 CUs in both directions (forward: rows x out_features,
        # grad-input: rows x in_features); with fewer the vendor library's smaller tiles fill the chip better
        row_tiles = (rows + 255) // 256
        full_round = row_tiles * min(self.out_features // 256, self.in_features // 256) >= TILED_GEMM_MIN_TILES
        return (x.shape[-1] == self.in_features and rows >= TILED_GEMM_MIN_ROWS and full_round
                and ops.tiled_weight_shape_ok(self.out_features, self.in_features, c.group_size))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.activation_fake_quantizer is not None:
            x = self.activation_fake_quantizer(x)
        if self._tiled_ok(x):
            return _TiledFakeQuantLinearFn.apply(x, self.weight, self.bias, self.weight_fake_quantizer)
        w = self.weight if self.weight_fake_quantizer is None else self.weight_fake_quantizer(self.weight)
        return F.linear(x, w, self.bias)

    def cross_entropy_sum(self, x: torch.Tensor, target: torch.Tensor, ignore_index: int = -100, scale: float = 1.0):
        """``scale * F.cross_entropy(self(x).float(), target, reduction="sum", ignore_index=ignore_index)`` for one chunk of
        rows, or None where this layer does not run on the library's own GEMM (the caller then composes it from
        ``self(x)``).  Same loss and gradients as the composition, without the pass that rescales the logits' gradient."""
        if self.bias is not None or self.weight_fake_quantizer is None:
            return None
        N = self.weight.shape[0]
        if N % 8 != 0 or N > 131072:
            return None
        if self.activation_fake_quantizer is not None:
            x = self.activation_fake_quantizer(x)
        if not self._tiled_ok(x):
            return None
        return _TiledFakeQuantLinearCrossEntropySumFn.apply(x, self.weight, self.weight_fake_quantizer, target, ignore_index, scale)

    def to_linear(self) -> nn.Linear:
        new = nn.Linear(self.in_features, self.out_features, self.bias is not None, device=self.weight.device,
                        dtype=self.weight.dtype)
        if self.weight.device != torch.device("meta"):
            new.weight = self.weight
            new.bias = self.bias
        return new

    @classmethod
    def from_linear(cls, mod: nn.Linear, activation_config=None, weight_config=None) -> "FakeQuantizedLinear":
        new = cls(mod.in_features, mod.out_features, mod.bias is not None, activation_config, weight_config,
                  device=mod.weight.device, dtype=mod.weight.dtype)
        if mod.weight.device != torch.device("meta"):
            new.weight = mod.weight
            new.bias = mod.bias
        return new


class Int8DynActInt4WeightQATLinear(FakeQuantizedLinear):
    """The linear ``Int8DynActInt4WeightQATQuantizer.prepare`` swaps in: per-token asymmetric int8 fake
    quantisation of the input, per-group symmetric int4 fake quantisation of the weight."""

    def __init__(
        self,
        in_features: int,
        out_features: int,
        bias: bool = False,
        device: Optional[torch.device] = None,
        groupsize: int = 256,
        precision: torch.dtype = torch.float32,
        scales_precision: torch.dtype = torch.float32,
    ) -> None:
        act = FakeQuantizeConfig(torch.int8, "per_token", is_symmetric=False, scale_precision=scales_precision)
        wgt = FakeQuantizeConfig(torch.int4, group_size=groupsize, is_symmetric=True, scale_precision=scales_precision)
        super().__init__(in_features, out_features, bias, act, wgt, device=device, dtype=precision)
        self.groupsize = groupsize
        self.precision = precision
        self.scales_precision = scales_precision

    def enable_fake_quant(self, enabled: bool = True):
        self.activation_fake_quantizer.enabled = enabled
        self.weight_fake_quantizer.enabled = enabled

    def disable_fake_quant(self):
        self.enable_fake_quant(False)


class Int8DynActInt4WeightLinear(nn.Module):
    """Result of ``convert``: int4 weight values held in int8 plus per-group scales and zeros; the input is
    quantised per token on the fly.  Forward reproduces the arithmetic the fake-quantised layer trained with."""

    def __init__(self, in_features: int, out_features: int, bias: bool = False, device=None, groupsize: int = 256,
                 precision: torch.dtype = torch.float32, scales_precision: torch.dtype = torch.float32) -> None:
        super().__init__()
        assert in_features % groupsize == 0, f"require in_features:{in_features} % groupsize:{groupsize} == 0"
        self.in_features = in_features
        self.out_features = out_features
        self.groupsize = groupsize
        self.precision = precision
        self.scales_precision = scales_precision
        self.register_buffer("weight", torch.zeros((out_features, in_features), dtype=torch.int8, device=device))
        self.register_buffer(
            "scales", torch.zeros((out_features, in_features // groupsize), dtype=scales_precision, device=device)
        )
        self.register_buffer(
            "zeros", torch.zeros((out_features, in_features // groupsize), dtype=scales_precision, device=device)
        )
        self.bias = nn.Parameter(torch.zeros(out_features, dtype=precision, device=device)) if bias else None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        x = x.to(self.precision)
        x_q, _, _ = ops.fq_per_token_int8_asym(x, want_qparams=False, qparam_dtype=self.scales_precision)
        w = ops.dequantize_per_group_int4(self.weight, self.scales, self.zeros, self.groupsize, self.precision)
        return F.linear(x_q, w, self.bias)


class Int8DynActInt4WeightQATQuantizer:
    """QAT quantizer for int8 dynamic per-token activations + int4 per-group symmetric weights.

    ``prepare(model)`` swaps every eligible ``nn.Linear`` for :class:`Int8DynActInt4WeightQATLinear`;
    ``convert(model)`` swaps those for :class:`Int8DynActInt4WeightLinear` holding real int4 values.
    """

    def __init__(
        self,
        groupsize: int = 256,
        padding_allowed: bool = False,
        precision: torch.dtype = torch.float32,
        scales_precision: torch.dtype = torch.float32,
    ) -> None:
        self.groupsize = groupsize
        self.padding_allowed = padding_allowed
        self.precision = precision
        self.scales_precision = scales_precision
        if padding_allowed:
            raise NotImplementedError("padding_allowed=True is not supported")

    def get_activation_fake_quantize_config(self) -> FakeQuantizeConfig:
        return FakeQuantizeConfig(torch.int8, "per_token", is_symmetric=False, scale_precision=self.scales_precision)

    def get_weight_fake_quantize_config(self) -> FakeQuantizeConfig:
        return FakeQuantizeConfig(torch.int4, group_size=self.groupsize, is_symmetric=True,
                                  scale_precision=self.scales_precision)

    def _eligible(self, lin: nn.Linear) -> bool:
        return lin.in_features % self.groupsize == 0

    def prepare(self, model: nn.Module, *args, **kwargs) -> nn.Module:
        for name, child in list(model.named_children()):
            if type(child) is nn.Linear and self._eligible(child):
                # built on the meta device (no second copy of the weight is ever allocated), then handed the original
                # Parameter objects: values, dtype, requires_grad and identity (optimizer state, tied weights) survive
                new = Int8DynActInt4WeightQATLinear(
                    child.in_features, child.out_features, child.bias is not None, device=torch.device("meta"),
                    groupsize=self.groupsize, precision=self.precision, scales_precision=self.scales_precision,
                )
                new.weight = child.weight
                new.bias = child.bias
                setattr(model, name, new)
            else:
                self.prepare(child)
        return model

    def convert(self, model: nn.Module, *args, **kwargs) -> nn.Module:
        for name, child in list(model.named_children()):
            if isinstance(child, Int8DynActInt4WeightQATLinear):
                new = Int8DynActInt4WeightLinear(
                    child.in_features, child.out_features, child.bias is not None, device=child.weight.device,
                    groupsize=child.groupsize, precision=child.weight.dtype, scales_precision=child.scales_precision,
                )
                q, scale, zeros = ops.quantize_per_group_int4(child.weight.detach(), child.groupsize, child.scales_precision)
                new.weight.copy_(q)
                new.scales.copy_(scale.to(child.scales_precision))
                new.zeros.copy_(zeros.to(child.scales_precision))
                if child.bias is not None:
                    new.bias = nn.Parameter(child.bias.detach(), requires_grad=False)
                setattr(model, name, new)
            else:
                self.convert(child)
        return model


# ---------------------------------------------------------------------------------------------------
# weight-only int4 ("4w-qat")
# ---------------------------------------------------------------------------------------------------
def _check_linear_int4_k(k: int, groupsize: int = 1, inner_k_tiles: Optional[int] = None) -> bool:
    """The shape rule of the weight-only int4 linear: K divisible by the group size and by 16 * inner_k_tiles."""
    ok = k % groupsize == 0
    if inner_k_tiles is not None:
        ok = ok and k % (inner_k_tiles * 16) == 0
    return ok


def _get_4w_weight_config(group_size: int, qparams_precision: torch.dtype) -> FakeQuantizeConfig:
    return FakeQuantizeConfig(
        dtype=torch.uint4, group_size=group_size, is_symmetric=False, is_dynamic=True, scale_precision=qparams_precision,
        zero_point_precision=qparams_precision, zero_point_domain=ZeroPointDomain.FLOAT,
    )


class Int4WeightOnlyQATLinear(FakeQuantizedLinear):
    """The linear ``Int4WeightOnlyQATQuantizer.prepare`` swaps in: the input passes unchanged, the weight is
    fake-quantised to uint4 per group (asymmetric, floating-point zero point, bf16 qparams)."""

    def __init__(
        self,
        in_features: int,
        out_features: int,
        bias: bool = False,
        device: Optional[torch.device] = None,
        groupsize: int = 256,
        inner_k_tiles: int = 8,
        precision: torch.dtype = torch.bfloat16,
        scales_precision: torch.dtype = torch.bfloat16,
    ) -> None:
        assert scales_precision == torch.bfloat16, "only bf16 is supported for scales"
        if not _check_linear_int4_k(in_features, groupsize, inner_k_tiles):
            raise ValueError("Padding for QAT 4w is not supported yet")
        self.groupsize = groupsize
        self.inner_k_tiles = inner_k_tiles
        self.precision = precision
        self.scales_precision = scales_precision
        super().__init__(in_features, out_features, bias, None, _get_4w_weight_config(groupsize, scales_precision),
                         device=device, dtype=precision)

    def enable_fake_quant(self, enabled: bool = True):
        self.weight_fake_quantizer.enabled = enabled

    def disable_fake_quant(self):
        self.enable_fake_quant(False)


class WeightOnlyInt4Linear(nn.Module):
    """Result of ``Int4WeightOnlyQATQuantizer.convert``: uint4 codes packed two per byte (``weight`` [N, K/2], even
    element in the high nibble) and ``scales_and_zeros`` [K/groupsize, N, 2] in bf16.  Forward rebuilds the dense
    weight the fake-quantised layer trained with and multiplies.

    The reference's converted module re-tiles the codes for one specific int4 matmul kernel
    (``aten._convert_weight_to_int4pack``); that opaque tiling is not reproduced, the plain packing is kept."""

    def __init__(self, in_features: int, out_features: int, bias: bool = False, device=None, groupsize: int = 128,
                 inner_k_tiles: int = 8, precision: torch.dtype = torch.bfloat16,
                 scales_precision: torch.dtype = torch.bfloat16) -> None:
        super().__init__()
        if not _check_linear_int4_k(in_features, groupsize, inner_k_tiles):
            raise ValueError("in_features must be divisible by groupsize and by 16 * inner_k_tiles")
        self.in_features = in_features
        self.out_features = out_features
        self.groupsize = groupsize
        self.inner_k_tiles = inner_k_tiles
        self.precision = precision
        self.scales_precision = scales_precision
        self.register_buffer("weight", torch.zeros((out_features, in_features // 2), dtype=torch.uint8, device=device))
        self.register_buffer(
            "scales_and_zeros",
            torch.zeros((in_features // groupsize, out_features, 2), dtype=scales_precision, device=device),
        )
        self.bias = nn.Parameter(torch.zeros(out_features, dtype=precision, device=device), requires_grad=False) if bias else None

    def dense_weight(self) -> torch.Tensor:
        sz = self.scales_and_zeros
        scale = sz[..., 0].t()
        zero = sz[..., 1].t()
        return ops.dequantize_per_group_uint4(self.weight, scale, zero, self.groupsize, self.precision)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return F.linear(x.to(self.precision), self.dense_weight(), self.bias)


class Int4WeightOnlyQATQuantizer:
    """QAT quantizer for the weight-only int4 scheme (mode ``"4w-qat"``).

    ``prepare(model)`` swaps every bias-free ``nn.Linear`` whose ``in_features`` fits the shape rule for
    :class:`Int4WeightOnlyQATLinear`; ``convert(model)`` swaps those for :class:`WeightOnlyInt4Linear`.
    """

    def __init__(
        self,
        groupsize: int = 256,
        inner_k_tiles: Optional[int] = 8,
        precision: torch.dtype = torch.bfloat16,
        scales_precision: torch.dtype = torch.bfloat16,
    ) -> None:
        assert inner_k_tiles in [2, 4, 8]
        assert groupsize in [32, 64, 128, 256]
        self.groupsize = groupsize
        self.inner_k_tiles = inner_k_tiles
        self.precision = precision
        self.scales_precision = scales_precision

    def get_weight_fake_quantize_config(self) -> FakeQuantizeConfig:
        return _get_4w_weight_config(self.groupsize, self.scales_precision)

    def prepare(self, model: nn.Module, *args, **kwargs) -> nn.Module:
        for name, child in list(model.named_children()):
            if (type(child) is nn.Linear and child.bias is None
                    and _check_linear_int4_k(child.in_features, self.groupsize, self.inner_k_tiles)):
                new = Int4WeightOnlyQATLinear(
                    child.in_features, child.out_features, False, device=torch.device("meta"), groupsize=self.groupsize,
                    inner_k_tiles=self.inner_k_tiles, precision=self.precision, scales_precision=self.scales_precision,
                )
                new.weight = child.weight  # the original Parameter: same dtype, same object
                setattr(model, name, new)
            else:
                self.prepare(child)
        return model

    def convert(self, model: nn.Module, *args, **kwargs) -> nn.Module:
        for name, child in list(model.named_children()):
            if isinstance(child, Int4WeightOnlyQATLinear):
                new = WeightOnlyInt4Linear(
                    child.in_features, child.out_features, False, device=child.weight.device, groupsize=child.groupsize,
                    inner_k_tiles=child.inner_k_tiles, precision=child.weight.dtype, scales_precision=child.scales_precision,
                )
                q, scale, zero = ops.quantize_per_group_uint4(child.weight.detach(), child.groupsize, child.scales_precision)
                new.weight.copy_(q)
                new.scales_and_zeros.copy_(torch.stack([scale.t(), zero.t()], dim=-1).to(child.scales_precision))
                setattr(model, name, new)
            else:
                self.convert(child)
        return model


# ---------------------------------------------------------------------------------------------------
# post-training quantisation with the same arithmetic (what recipes/quantize.py runs for the non-QAT modes)
# ---------------------------------------------------------------------------------------------------
def quantize_linears_8da4w(model: nn.Module, groupsize: int) -> nn.Module:
    """Swap every ``nn.Linear`` for :class:`Int8DynActInt4WeightLinear` holding the int4 codes of its weight."""
    for name, child in list(model.named_children()):
        if type(child) is nn.Linear:
            if child.in_features % groupsize != 0:
                raise ValueError(f"{name}: in_features ({child.in_features}) must be divisible by groupsize ({groupsize})")
            new = Int8DynActInt4WeightLinear(
                child.in_features, child.out_features, child.bias is not None, device=child.weight.device,
                groupsize=groupsize, precision=child.weight.dtype, scales_precision=torch.float32,
            )
            q, scale, zeros = ops.quantize_per_group_int4(child.weight.detach(), groupsize)
            new.weight.copy_(q)
            new.scales.copy_(scale)
            new.zeros.copy_(zeros)
            if child.bias is not None:
                new.bias = nn.Parameter(child.bias.detach(), requires_grad=False)
            setattr(model, name, new)
        else:
            quantize_linears_8da4w(child, groupsize)
    return model


def quantize_linears_4w(model: nn.Module, groupsize: int, inner_k_tiles: int) -> nn.Module:
    """Swap every ``nn.Linear`` for :class:`WeightOnlyInt4Linear` holding the uint4 codes of its weight."""
    for name, child in list(model.named_children()):
        if type(child) is nn.Linear:
            if not _check_linear_int4_k(child.in_features, groupsize, inner_k_tiles):
                raise ValueError(f"{name}: in_features ({child.in_features}) must be divisible by groupsize ({groupsize}) "
                                 f"and by 16 * inner_k_tiles ({16 * inner_k_tiles})")
            new = WeightOnlyInt4Linear(
                child.in_features, child.out_features, child.bias is not None, device=child.weight.device, groupsize=groupsize,
                inner_k_tiles=inner_k_tiles, precision=child.weight.dtype, scales_precision=torch.bfloat16,
            )
            q, scale, zero = ops.quantize_per_group_uint4(child.weight.detach(), groupsize, torch.bfloat16)
            new.weight.copy_(q)
            new.scales_and_zeros.copy_(torch.stack([scale.t(), zero.t()], dim=-1).to(torch.bfloat16))
            if child.bias is not None:
                new.bias = nn.Parameter(child.bias.detach(), requires_grad=False)
            setattr(model, name, new)
        else:
            quantize_linears_4w(child, groupsize, inner_k_tiles)
    return model
