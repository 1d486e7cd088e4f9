"""CPU oracle for the QAT fake-quantisation arithmetic (8da4w: int8 dynamic per-token activations, int4
per-group symmetric weights).

TEST INFRASTRUCTURE ONLY — never imported by the shipped package.

Eager-PyTorch restatement of what the reference runs through ``torchao.quantization.qat``:

* ``fq_per_token_int8_asym``   <- ``FakeQuantizer`` built from ``FakeQuantizeConfig(torch.int8, "per_token",
  is_symmetric=False)``; reference: ``torchtune/modules/peft/lora.py:232,258``, created for every linear by
  ``Int8DynActInt4WeightQATQuantizer.prepare`` (``recipes/qat_single_device.py:378-386``).
* ``fq_per_group_int4_sym``    <- ``FakeQuantizer`` built from ``FakeQuantizeConfig(torch.int4, group_size=g,
  is_symmetric=True)``; reference: ``torchtune/modules/peft/lora.py:245,259``.
* ``quantize_per_group_int4``  <- ``quantizer.convert(model)`` (``recipes/quantize.py:92``).
* ``fake_quantized_linear``    <- ``FakeQuantizedLinear.forward``: ``F.linear(fq(x), fq(W))`` with the
  straight-through estimator in backward; the prose description is at
  ``docs/source/tutorials/qat_finetune.rst:40-50``.

* ``fq_per_group_uint4_asym`` / ``quantize_per_group_uint4`` / ``dequantize_per_group_uint4`` <- the weight-only
  ``Int4WeightOnlyQATQuantizer`` (``torchtune/training/quantization.py:27,125-127``, mode ``"4w-qat"``): group-wise
  asymmetric uint4 with a floating-point zero point, qparams in bf16.

Parity status: PARITY UNPINNED against torchao itself (not importable here; the reference holds no vectors
for these functions).  Pinned instead by closed forms and invariants in tests/test_oracle_fake_quant.py
(scale = (max-min)/255 and the zero-point formula on hand-built rows, outputs on the scale*(q-zp) grid,
idempotence for fixed qparams, exhaustive tiny cases), by the independent C restatement oracle/nf4_ref.c, and by
agreement (qparams, codes and values, bit for bit on fp32 inputs) with the implementation of the same per-token /
per-group scheme that ships inside PyTorch itself, ``torch.ops.quantized_decomposed``
(``torch/ao/quantization/fx/_decomposed.py``).

Numerics: qparams are computed in fp32 from the fp32-promoted input (and cast to the config's ``scale_precision``
— float32 by default, the reference's documented setting — before they are used); eps = finfo(float32).eps;
``round`` is round-half-to-even; the dequantised value is ``(q - zp)`` cast to the input dtype, times the fp32
scale, cast back to the input dtype.  The backward mask ``(q >= qmin) & (q <= qmax)`` is evaluated on the
clamped ``q`` and is therefore all ones: the gradient passes straight through.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

_EPS = torch.finfo(torch.float32).eps


def choose_qparams_per_token_asym(x: torch.Tensor, eps: float = None):
    """int8 asymmetric qparams for each row of the last dimension -> (scale fp32 [...,1], zero_point int32 [...,1])."""
    qmin, qmax = -128, 127
    xf = x.to(torch.float32)
    mn = torch.amin(xf, dim=-1, keepdim=True)
    mx = torch.amax(xf, dim=-1, keepdim=True)
    mn_neg = torch.min(mn, torch.zeros_like(mn))
    mx_pos = torch.max(mx, torch.zeros_like(mx))
    scale = (mx_pos - mn_neg) / float(qmax - qmin)
    scale = scale.clamp(min=_EPS if eps is None else eps)
    descaled_min = mn_neg / scale
    descaled_max = mx_pos / scale
    zp_from_min_err = qmin + descaled_min
    zp_from_max_err = qmax + descaled_max
    zp = torch.where(zp_from_min_err + zp_from_max_err > 0, qmin - descaled_min, qmax - descaled_max)
    zp = torch.clamp(zp, qmin, qmax).round()
    return scale, zp.to(torch.int32)


def _fake_quantize(x: torch.Tensor, scale: torch.Tensor, zp: torch.Tensor, qmin: int, qmax: int):
    q = torch.clamp(torch.round(x * (1.0 / scale)) + zp, qmin, qmax)
    dq = (q.to(torch.int32) - zp.to(torch.int32)).to(x.dtype)
    dq = (dq * scale).to(x.dtype)
    return q, dq


def _to_scale_precision(scale: torch.Tensor, scale_dtype: torch.dtype) -> torch.Tensor:
    """The qparams are cast to the config's ``scale_precision`` before use; the value is widened back for the arithmetic."""
    return scale.to(scale_dtype).to(torch.float32)


def fq_per_token_int8_asym(x: torch.Tensor, scale_dtype: torch.dtype = torch.float32, eps: float = None):
    """returns (fake-quantised x, scale [rows] fp32, zero_point [rows] int32); with ``scale_dtype=bfloat16`` the scale is
    rounded to bf16 after the zero point has been chosen, and the rounded scale quantises and dequantises"""
    scale, zp = choose_qparams_per_token_asym(x, eps)
    scale = _to_scale_precision(scale, scale_dtype)
    _, dq = _fake_quantize(x, scale, zp, -128, 127)
    return dq, scale.reshape(-1), zp.reshape(-1)


def choose_qparams_per_group_sym(w: torch.Tensor, group_size: int, eps: float = None):
    """int4 symmetric qparams per group of `group_size` along the last dim -> scale fp32 [rows, K/g]."""
    qmin, qmax = -8, 7
    rows, K = w.shape
    g = w.to(torch.float32).view(rows, K // group_size, group_size)
    mn = torch.amin(g, dim=-1)
    mx = torch.amax(g, dim=-1)
    mn_neg = torch.min(mn, torch.zeros_like(mn))
    mx_pos = torch.max(mx, torch.zeros_like(mx))
    amax = torch.max(-mn_neg, mx_pos)
    scale = amax / (float(qmax - qmin) / 2)
    return scale.clamp(min=_EPS if eps is None else eps)


def fq_per_group_int4_sym(w: torch.Tensor, group_size: int, scale_dtype: torch.dtype = torch.float32, eps: float = None):
    """returns (fake-quantised w, scale [rows, K/g] fp32)"""
    rows, K = w.shape
    scale = _to_scale_precision(choose_qparams_per_group_sym(w, group_size, eps), scale_dtype)
    wg = w.view(rows, K // group_size, group_size)
    zp = torch.zeros_like(scale, dtype=torch.int32)
    _, dq = _fake_quantize(wg, scale[..., None], zp[..., None], -8, 7)
    return dq.reshape(rows, K), scale


def quantize_per_group_int4(w: torch.Tensor, group_size: int, scale_dtype: torch.dtype = torch.float32, eps: float = None):
    """convert(): returns (int8 tensor of int4 values [rows,K], scale [rows,K/g] fp32, zeros [rows,K/g] fp32)"""
    rows, K = w.shape
    scale = _to_scale_precision(choose_qparams_per_group_sym(w, group_size, eps), scale_dtype)
    wg = w.view(rows, K // group_size, group_size)
    q = torch.clamp(torch.round(wg * (1.0 / scale[..., None])), -8, 7).to(torch.int8)
    return q.reshape(rows, K), scale, torch.zeros_like(scale)


# ---- weight-only int4 ("4w-qat": asymmetric uint4 with a floating-point zero point) --------------------------
def choose_qparams_per_group_uint4_asym(w: torch.Tensor, group_size: int, qparam_dtype: torch.dtype = torch.bfloat16,
                                        min_scale: float = 1e-6, clamp_range_first: bool = False):
    """Group-wise affine qparams of the weight-only int4 scheme, computed op by op in the dtype of ``w`` (the
    eager sequence rounds after every operation) and then cast to ``qparam_dtype``:
    ``scale = clamp((max - min) / 15, 1e-6)``, ``zero_point = min + scale * 8``.  The group extrema are NOT widened
    to include 0.  -> (scale, zero_point), each [rows, K/g] in ``qparam_dtype``.
    ``clamp_range_first``: the other order found among versions of the scheme, ``scale = clamp(max - min, min_scale) / 15``."""
    rows, K = w.shape
    g = w.view(rows, K // group_size, group_size)
    mn = torch.amin(g, dim=-1)
    mx = torch.amax(g, dim=-1)
    if clamp_range_first:
        scale = torch.clamp(mx - mn, min=min_scale) / 15.0
    else:
        scale = (mx - mn) / 15.0
        scale = torch.clamp(scale, min=min_scale)
    zero = mn + scale * 8.0
    return scale.to(qparam_dtype), zero.to(qparam_dtype)


def _uint4_codes(w: torch.Tensor, scale: torch.Tensor, zero: torch.Tensor, group_size: int) -> torch.Tensor:
    rows, K = w.shape
    g = w.view(rows, K // group_size, group_size)
    sc = scale.to(w.dtype)[..., None]
    zp = zero.to(w.dtype)[..., None]
    lowest = zp - sc * 8.0
    return torch.clamp(torch.round((g - lowest) / sc), 0, 15)


def fq_per_group_uint4_asym(w: torch.Tensor, group_size: int, qparam_dtype: torch.dtype = torch.bfloat16,
                            min_scale: float = 1e-6, clamp_range_first: bool = False):
    """returns (fake-quantised w, scale [rows, K/g], zero_point [rows, K/g]) — qparams in ``qparam_dtype``."""
    rows, K = w.shape
    scale, zero = choose_qparams_per_group_uint4_asym(w, group_size, qparam_dtype, min_scale, clamp_range_first)
    q = _uint4_codes(w, scale, zero, group_size)
    dq = (q - 8.0) * scale.to(w.dtype)[..., None]
    dq = dq + zero.to(w.dtype)[..., None]
    return dq.reshape(rows, K), scale, zero


def quantize_per_group_uint4(w: torch.Tensor, group_size: int, qparam_dtype: torch.dtype = torch.bfloat16,
                             min_scale: float = 1e-6, clamp_range_first: bool = False):
    """convert() of the weight-only scheme: (uint8 [rows, K/2], even element in the high nibble; scale; zero_point)."""
    rows, K = w.shape
    scale, zero = choose_qparams_per_group_uint4_asym(w, group_size, qparam_dtype, min_scale, clamp_range_first)
    q = _uint4_codes(w, scale, zero, group_size).reshape(rows, K).to(torch.uint8)
    return (q[:, ::2] << 4) | q[:, 1::2], scale, zero


def dequantize_per_group_uint4(packed: torch.Tensor, scale: torch.Tensor, zero: torch.Tensor, group_size: int,
                               dtype: torch.dtype) -> torch.Tensor:
    rows, half = packed.shape
    q = torch.stack([packed >> 4, packed & 15], dim=-1).reshape(rows, half * 2).to(dtype)
    g = q.view(rows, -1, group_size)
    dq = (g - 8.0) * scale.to(dtype)[..., None]
    dq = dq + zero.to(dtype)[..., None]
    return dq.reshape(rows, half * 2)


class _STE(torch.autograd.Function):
    """y = fq(x) in forward, dy/dx = 1 in backward (the all-ones mask of the reference)."""

    @staticmethod
    def forward(ctx, x, fq):
        return fq

    @staticmethod
    def backward(ctx, g):
        return g, None


def fake_quantized_linear(x: torch.Tensor, w: torch.Tensor, group_size: int, bias=None) -> torch.Tensor:
    """FakeQuantizedLinear.forward with both fake quantisers enabled; differentiable w.r.t. x and w."""
    x2 = x.reshape(-1, x.shape[-1])
    x_fq = _STE.apply(x2, fq_per_token_int8_asym(x2.detach())[0]).reshape(x.shape)
    w_fq = _STE.apply(w, fq_per_group_int4_sym(w.detach(), group_size)[0])
    return F.linear(x_fq, w_fq, bias)
