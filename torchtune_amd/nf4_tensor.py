"""``NF4Tensor``, ``to_nf4`` and ``linear_nf4`` backed by the HIP kernels.

This module is the seam the reference binds at: torchtune imports ``to_nf4`` / ``NF4Tensor`` from
``torchao.quantization`` and ``linear_nf4`` / ``implements`` from
``torchao.quantization.quantize_.workflows.nf4.nf4_tensor`` (``torchtune/modules/peft/lora.py:15-16``,
``torchtune/modules/low_precision/nf4_linear.py:12-13``, ``torchtune/modules/common_utils.py:19``,
``torchtune/modules/low_precision/_register_nf4_dispatch_ops.py:8-9``).  The names, signatures and the eight
public attributes (``tests/torchtune/modules/low_precision/test_nf4_dispatch_registration.py:22-31``) are
kept; the arithmetic runs in ``libtorchtune_amd.so``.

Tensors that live on the CPU are staged through the GPU for quantise / dequantise (the kernels are the only
implementation); with no GPU present those calls raise.
"""
from __future__ import annotations

import math
import weakref
from typing import Any, Callable, Dict, Iterable, Optional

import torch
import torch.nn.functional as F

from . import ops

aten = torch.ops.aten

# Default granularity of to_nf4: 64-element blocks, 256 block scalers per double-quantisation group.
DEFAULT_BLOCK_SIZE = 64
DEFAULT_SCALER_BLOCK_SIZE = 256

# Keep a transposed copy of the codes for the grad-input GEMM (see NF4Tensor.backward_copy).
BACKWARD_COPY = True

NF4_TABLE = (
    -1.0,
    -0.6961928009986877,
    -0.5250730514526367,
    -0.39491748809814453,
    -0.28444138169288635,
    -0.18477343022823334,
    -0.09105003625154495,
    0.0,
    0.07958029955625534,
    0.16093020141124725,
    0.24611230194568634,
    0.33791524171829224,
    0.44070982933044434,
    0.5626170039176941,
    0.7229568362236023,
    1.0,
)

NF4_OPS_TABLE: Dict[Any, Callable] = {}
NF4_TORCH_FUNCTIONS: Dict[Any, Callable] = {}

_INNER_TENSORS = ("quantized_scalers", "quantization_factor", "scaler_mean", "quantized_data", "nf4")


# Writes into an NF4 tensor happen inside __torch_dispatch__, where the in-place version counters of the inner tensors do
# not advance, and an alias (``param.data``, ``param.detach()``) has inner tensor objects of its own over the same
# storage.  The derived-data caches (block scalers, transposed copy) are therefore keyed on a generation number kept
# per storage address of the scaler bytes: ``copy_`` bumps it, so every alias sees its cache go stale.
_WRITE_GENERATION: Dict[int, int] = {}


def _generation(qs: torch.Tensor) -> int:
    return _WRITE_GENERATION.get(qs.untyped_storage().data_ptr(), 0) if qs.device.type != "meta" else 0


def _bump_generation(qs: torch.Tensor) -> None:
    if qs.device.type != "meta":
        ptr = qs.untyped_storage().data_ptr()
        _WRITE_GENERATION[ptr] = _WRITE_GENERATION.get(ptr, 0) + 1


def implements(aten_ops: Iterable[Any]):
    """Register a ``__torch_dispatch__`` handler for NF4Tensor.  The handler is called as
    ``handler(func, args, kwargs)`` with the positional arguments still packed in one tuple, which is the
    convention ``torchtune/modules/low_precision/_register_nf4_dispatch_ops.py:12-20`` relies on."""

    def decorator(fn):
        for op in aten_ops:
            NF4_OPS_TABLE[op] = fn
        return fn

    return decorator


def implements_torch_function(torch_fn):
    def decorator(fn):
        NF4_TORCH_FUNCTIONS[torch_fn] = fn
        return fn

    return decorator


def shape_and_dtype(weight: "NF4Tensor"):
    """``(tuple(weight.shape), weight.dtype)`` for the per-call host code.  ``shape`` / ``dtype`` of a tensor subclass are
    routed through ``__torch_function__`` (microseconds each, a dozen reads per layer call), so the pair is kept on the
    packed-data tensor object, with a weak reference to the NF4 tensor it describes.  (Not on the NF4 tensor itself: the
    reference pins the exact key set of its ``__dict__``,
    tests/torchtune/modules/low_precision/test_nf4_dispatch_registration.py:22-35, and ``torch.utils.swap_tensors``
    refuses tensors whose slots differ.)"""
    packed = weight.quantized_data
    memo = packed.__dict__.get("_ttamd_outer")
    if memo is not None and memo[0]() is weight:
        return memo[1], memo[2]
    shape, dtype = tuple(weight.shape), weight.dtype
    try:
        packed._ttamd_outer = (weakref.ref(weight), shape, dtype)
    except TypeError:
        pass
    return shape, dtype


def _compute_device(t: torch.Tensor) -> torch.device:
    """Device the kernels run on for tensor ``t``: its own if it is on a GPU, otherwise the current GPU."""
    if t.is_cuda:
        return t.device
    if t.device.type == "cpu" and torch.cuda.is_available():
        return torch.device("cuda", torch.cuda.current_device())
    raise RuntimeError(
        f"NF4 quantise/dequantise of a tensor on '{t.device}' needs an AMD GPU: torchtune_amd computes only "
        "through its HIP kernels and no GPU is visible."
    )


class NF4Tensor(torch.Tensor):
    """4-bit NormalFloat weight with double-quantised block scalers.

    Behaves like a frozen tensor of the original shape and dtype.  ``.to(dtype)`` and
    ``get_original_weight()`` return the dequantised dense tensor; ``.to(device)`` / ``.cpu()`` move the
    packed representation; ``copy_`` from a dense tensor re-quantises in place.
    """

    @staticmethod
    def __new__(
        cls,
        shape,
        dtype: torch.dtype,
        block_size: int,
        n_blocks: int,
        scaler_block_size: int,
        quantized_scalers: torch.Tensor,
        quantization_factor: torch.Tensor,
        scaler_mean: torch.Tensor,
        quantized_data: torch.Tensor,
        nf4: torch.Tensor,
        requires_grad: bool = False,
    ):
        return torch.Tensor._make_wrapper_subclass(
            cls,
            torch.Size(shape),
            dtype=dtype,
            device=quantized_data.device,
            requires_grad=requires_grad,
        )

    def __init__(
        self,
        shape,
        dtype: torch.dtype,
        block_size: int,
        n_blocks: int,
        scaler_block_size: int,
        quantized_scalers: torch.Tensor,
        quantization_factor: torch.Tensor,
        scaler_mean: torch.Tensor,
        quantized_data: torch.Tensor,
        nf4: torch.Tensor,
        requires_grad: bool = False,
    ):
        self.block_size = block_size
        self.n_blocks = n_blocks
        self.scaler_block_size = scaler_block_size
        self.quantized_scalers = quantized_scalers
        self.quantization_factor = quantization_factor
        self.scaler_mean = scaler_mean
        self.quantized_data = quantized_data
        self.nf4 = nf4

    # ---- construction ------------------------------------------------------------------------------
    @classmethod
    @torch.no_grad()
    def from_tensor(cls, tensor: torch.Tensor, block_size: int, scaler_block_size: int) -> "NF4Tensor":
        assert tensor.dim() <= 2, f"expect input tensor dim <= 2 but got dim = {tensor.dim()}"
        assert tensor.numel() % block_size == 0, (
            f"Input tensor must be divisible by block size, got {tensor.numel()} and {block_size}"
        )
        assert tensor.is_contiguous(), "Input tensor must be contiguous!"
        n_blocks = tensor.numel() // block_size
        assert n_blocks % scaler_block_size == 0, (
            f"Number of blocks ({n_blocks}) must be divisible by scaler_block_size ({scaler_block_size})"
        )
        home = tensor.device
        dev = _compute_device(tensor)
        w = tensor.detach().to(dev)
        qdata, qscalers, qfactor, mean = ops.nf4_quantize(w, block_size, scaler_block_size)
        nf4 = torch.tensor(NF4_TABLE, dtype=tensor.dtype, device=dev)
        inner = [qscalers, qfactor, mean, qdata, nf4]
        if home != dev:
            inner = [t.to(home) for t in inner]
        return cls(tensor.shape, tensor.dtype, block_size, n_blocks, scaler_block_size, *inner)

    def _rewrap(self, inner: Dict[str, torch.Tensor], **overrides) -> "NF4Tensor":
        return NF4Tensor(
            overrides.get("shape", self.shape),
            self.dtype,
            self.block_size,
            self.n_blocks,
            self.scaler_block_size,
            inner["quantized_scalers"],
            inner["quantization_factor"],
            inner["scaler_mean"],
            inner["quantized_data"],
            inner["nf4"],
            requires_grad=overrides.get("requires_grad", False),
        )

    def _map_inner(self, fn) -> Dict[str, torch.Tensor]:
        return {name: fn(getattr(self, name)) for name in _INNER_TENSORS}

    # ---- dequantisation ----------------------------------------------------------------------------
    @torch.no_grad()
    def get_original_weight(self, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The dequantised weight in the original dtype and shape.  With ``out`` (same dtype and element count, on
        the weight's GPU or in pinned host memory) the kernel stores into it directly; for host memory the caller
        synchronises the current stream before reading the values."""
        home = self.quantized_data.device
        dev = _compute_device(self.quantized_data)
        parts = [self.quantized_data, self.quantized_scalers, self.quantization_factor, self.scaler_mean]
        if home != dev:
            parts = [t.to(dev) for t in parts]
        if out is not None:
            ops.nf4_dequantize(*parts, self.shape, self.block_size, self.scaler_block_size, out=out)
            return out
        out = ops.nf4_dequantize(*parts, self.shape, self.block_size, self.scaler_block_size)
        return out if home == dev else out.to(home)

    @torch.no_grad()
    def block_scalers(self) -> torch.Tensor:
        """Dequantised per-block scalers as fp32 [n_blocks] on the GPU, cached while the scaler tensors are
        unchanged (the cache rides on the ``quantized_scalers`` tensor object and is keyed by the in-place
        version counters of the three scaler tensors and the write generation of their storage)."""
        qs = self.quantized_scalers
        key = (qs._version, self.quantization_factor._version, self.scaler_mean._version, qs.data_ptr(), _generation(qs))
        cached = getattr(qs, "_ttamd_block_scalers", None)
        if cached is not None and cached[0] == key:
            return cached[1]
        val = ops.nf4_block_scalers(qs, self.quantization_factor, self.scaler_mean, self.scaler_block_size)
        qs._ttamd_block_scalers = (key, val)
        return val

    @torch.no_grad()
    def backward_copy(self):
        """(codes re-packed along N, block scalers transposed) for the grad-input GEMM, or None when disabled.

        Derived data for a 2-D bf16 tensor with 64-element blocks, cached like ``block_scalers`` (same key).  It
        costs another 0.5625 B per element of device memory; set ``torchtune_amd.nf4_tensor.BACKWARD_COPY = False``
        to trade that memory for a slower grad-input GEMM that transposes the weight tile on the fly."""
        if not BACKWARD_COPY:
            return None
        qs = self.quantized_scalers
        key = (qs._version, self.quantization_factor._version, self.scaler_mean._version, self.quantized_data._version,
               qs.data_ptr(), _generation(qs))
        cached = getattr(qs, "_ttamd_backward_copy", None)
        if cached is not None and cached[0] == key:
            return cached[1]
        val = ops.nf4_transpose_for_backward(self.quantized_data, self.block_scalers(), self.shape[0], self.shape[1])
        qs._ttamd_backward_copy = (key, val)
        return val

    def resident_tiles(self):
        """The expanded weight a many-token forward left behind and ``keep_resident_tiles`` stored, while the weight is
        unchanged (``ops.RESIDENT_TILES_MAX_BYTES``); else None."""
        cached = getattr(self.quantized_scalers, "_ttamd_tiles", None)
        return cached[1] if cached is not None and cached[0] == _tiles_key(self) else None

    def keep_resident_tiles(self, tiles: torch.Tensor) -> bool:
        """Stores a forward call's tiles with the weight if the budget admits them; True when stored."""
        if not ops.resident_tiles_admit(tiles):
            return False
        self.quantized_scalers._ttamd_tiles = (_tiles_key(self), tiles)
        return True

    def backward_copy_for(self, tokens: int, forward: bool):
        """The transposed copy a GEMM call over ``tokens`` rows would use: None when the library serves that call from the
        weight expanded once per call (many tokens; it then reads the weight's own codes, so a purely many-token
        training run never builds the copy), otherwise ``backward_copy()``."""
        N, K = shape_and_dtype(self)[0]
        n_out, k_contract = (N, K) if forward else (K, N)
        if ops.gemm_expands_weight(tokens, n_out, k_contract):
            return None
        return self.backward_copy()

    # ---- tensor-subclass protocol --------------------------------------------------------------------
    def __tensor_flatten__(self):
        ctx = {
            "block_size": self.block_size,
            "n_blocks": self.n_blocks,
            "scaler_block_size": self.scaler_block_size,
            "shape": tuple(self.shape),
            "dtype": self.dtype,
        }
        return list(_INNER_TENSORS), ctx

    @staticmethod
    def __tensor_unflatten__(inner_tensors, ctx, outer_size=None, outer_stride=None):
        return NF4Tensor(
            ctx["shape"],
            ctx["dtype"],
            ctx["block_size"],
            ctx["n_blocks"],
            ctx["scaler_block_size"],
            inner_tensors["quantized_scalers"],
            inner_tensors["quantization_factor"],
            inner_tensors["scaler_mean"],
            inner_tensors["quantized_data"],
            inner_tensors["nf4"],
        )

    def __repr__(self) -> str:
        return (
            f"NF4Tensor(shape={tuple(self.shape)}, dtype={self.dtype}, device={self.device}, "
            f"block_size={self.block_size}, scaler_block_size={self.scaler_block_size})"
        )

    __str__ = __repr__

    @classmethod
    def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        handler = NF4_OPS_TABLE.get(func)
        if handler is None:
            raise NotImplementedError(f"NF4Tensor does not support {func}")
        return handler(func, args, kwargs)

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        handler = NF4_TORCH_FUNCTIONS.get(func)
        if handler is not None:
            return handler(*args, **kwargs)
        with torch._C.DisableTorchFunctionSubclass():
            return func(*args, **kwargs)


def _tiles_key(w: "NF4Tensor"):
    qs = w.quantized_scalers
    return (qs._version, w.quantization_factor._version, w.scaler_mean._version, w.quantized_data._version, qs.data_ptr(),
            w.quantized_data.data_ptr(), _generation(qs))


def resident_group_tiles(weights, swiglu: bool):
    """``(tiles, paired)`` that ``keep_resident_group_tiles`` stored for exactly these weights (unchanged since) and this
    kind of group call, or None."""
    cached = getattr(weights[0].quantized_scalers, "_ttamd_group_tiles", None)
    if cached is not None and cached[0] == (bool(swiglu),) + tuple(_tiles_key(w) for w in weights):
        return cached[1], cached[2]
    return None


def keep_resident_group_tiles(weights, swiglu: bool, tiles: torch.Tensor, paired: bool) -> bool:
    """Stores a group forward's tiles with the group's first weight if the budget admits them; True when stored."""
    if not ops.resident_tiles_admit(tiles):
        return False
    weights[0].quantized_scalers._ttamd_group_tiles = ((bool(swiglu),) + tuple(_tiles_key(w) for w in weights), tiles, paired)
    return True


# ---- aten-level behaviour -----------------------------------------------------------------------------
def _carry_cache(src: NF4Tensor, dst: NF4Tensor) -> None:
    cached = getattr(src.quantized_scalers, "_ttamd_block_scalers", None)
    if cached is not None and dst.quantized_scalers.data_ptr() == src.quantized_scalers.data_ptr():
        key = (dst.quantized_scalers._version, dst.quantization_factor._version, dst.scaler_mean._version,
               dst.quantized_scalers.data_ptr(), _generation(dst.quantized_scalers))
        if key == cached[0]:
            dst.quantized_scalers._ttamd_block_scalers = cached


@implements([aten.detach.default, aten.alias.default])
def _nf4_detach(func, args, kwargs):
    src = args[0]
    out = src._rewrap(src._map_inner(lambda t: func(t)))
    _carry_cache(src, out)
    return out


@implements([aten.clone.default])
def _nf4_clone(func, args, kwargs):
    # same behaviour as the override in torchtune/modules/low_precision/_register_nf4_dispatch_ops.py:12-20:
    # a clone is a re-quantisation of the dequantised weight with the default granularity
    return to_nf4(args[0].get_original_weight())


@implements([aten.copy_.default])
def _nf4_copy_(func, args, kwargs):
    dst, src = args[0], args[1]
    if not isinstance(dst, NF4Tensor):
        # dense.copy_(nf4): materialise
        return func(dst, src.get_original_weight(), **kwargs)
    # in-place writes issued from inside __torch_dispatch__ do not advance the version counters, so the caches of
    # this tensor object are dropped and the storage's write generation is bumped for those of its aliases
    dst.quantized_scalers._ttamd_block_scalers = None
    dst.quantized_scalers._ttamd_backward_copy = None
    dst.quantized_scalers._ttamd_tiles = None
    dst.quantized_scalers._ttamd_group_tiles = None
    _bump_generation(dst.quantized_scalers)
    if isinstance(src, NF4Tensor):
        same_meta = (
            src.block_size == dst.block_size
            and src.scaler_block_size == dst.scaler_block_size
            and src.n_blocks == dst.n_blocks
            and src.shape == dst.shape
            and src.dtype == dst.dtype
        )
        if same_meta:
            for name in _INNER_TENSORS:
                getattr(dst, name).copy_(getattr(src, name), **kwargs)
            return dst
        src = src.get_original_weight()
    if src.shape != dst.shape:
        src = src.expand(dst.shape)
    fresh = NF4Tensor.from_tensor(
        src.detach().to(device=dst.device, dtype=dst.dtype).contiguous(), dst.block_size, dst.scaler_block_size
    )
    for name in _INNER_TENSORS:
        getattr(dst, name).copy_(getattr(fresh, name))
    return dst


@implements([aten._to_copy.default])
def _nf4_to_copy(func, args, kwargs):
    src = args[0]
    dtype = kwargs.get("dtype")
    device = kwargs.get("device")
    if dtype is not None and dtype != src.dtype:
        dense = src.get_original_weight().to(dtype)
        return dense if device is None else dense.to(device)
    if device is None:
        device = src.device
    non_blocking = kwargs.get("non_blocking", False)
    return src._rewrap(src._map_inner(lambda t: t.to(device, non_blocking=non_blocking)))


@implements([aten.is_pinned.default])
def _nf4_is_pinned(func, args, kwargs):
    return all(getattr(args[0], name).is_pinned() for name in _INNER_TENSORS)


@implements([aten._pin_memory.default])
def _nf4_pin_memory(func, args, kwargs):
    return args[0]._rewrap(args[0]._map_inner(lambda t: func(t)))


@implements([aten.empty_like.default])
def _nf4_empty_like(func, args, kwargs):
    src = args[0]
    inner_kwargs = {k: v for k, v in kwargs.items() if k in ("device", "pin_memory") and v is not None}
    return src._rewrap(src._map_inner(lambda t: torch.empty_like(t, **inner_kwargs)))


@implements([aten.equal.default])
def _nf4_equal(func, args, kwargs):
    a, b = args[0], args[1]
    if not (isinstance(a, NF4Tensor) and isinstance(b, NF4Tensor)):
        return False
    return (
        a.shape == b.shape
        and a.block_size == b.block_size
        and a.scaler_block_size == b.scaler_block_size
        and all(torch.equal(getattr(a, n), getattr(b, n)) for n in _INNER_TENSORS)
    )


# ---- torch-function-level behaviour -------------------------------------------------------------------
def _parse_to_args(args, kwargs):
    """Extract (device, dtype, non_blocking) from the argument forms of Tensor.to."""
    device = kwargs.get("device")
    dtype = kwargs.get("dtype")
    non_blocking = kwargs.get("non_blocking", False)
    for a in args:
        if isinstance(a, torch.dtype):
            dtype = a
        elif isinstance(a, (torch.device, str, int)) and not isinstance(a, bool):
            device = torch.device(a) if not isinstance(a, int) else torch.device("cuda", a)
        elif isinstance(a, torch.Tensor):
            device, dtype = a.device, a.dtype
        elif isinstance(a, bool):
            non_blocking = a  # first bool positional after device/dtype is non_blocking
    return device, dtype, non_blocking


@implements_torch_function(torch.Tensor.to)
def _nf4_function_to(*args, **kwargs):
    tensor = args[0]
    device, dtype, non_blocking = _parse_to_args(args[1:], kwargs)
    if dtype is not None:
        # Tensor.to(dtype) always materialises the dense weight, also when dtype == tensor.dtype
        # (torchtune/modules/common_utils.py:57 relies on that to strip NF4 from state dicts)
        dense = tensor.get_original_weight()
        if dtype != dense.dtype:
            dense = dense.to(dtype)
        return dense if device is None else dense.to(device, non_blocking=non_blocking)
    if device is None:
        return tensor
    out = tensor._rewrap(
        tensor._map_inner(lambda t: t.to(device, non_blocking=non_blocking)), requires_grad=tensor.requires_grad
    )
    return out


@implements_torch_function(torch.Tensor.cpu)
def _nf4_function_cpu(*args, **kwargs):
    return _nf4_function_to(args[0], torch.device("cpu"))


@implements_torch_function(torch.Tensor.cuda)
def _nf4_function_cuda(*args, **kwargs):
    device = args[1] if len(args) > 1 else kwargs.get("device")
    if device is None:
        device = torch.device("cuda", torch.cuda.current_device())
    return _nf4_function_to(args[0], device)


@implements_torch_function(F.linear)
def _nf4_function_linear(*args, **kwargs):
    inp = args[0] if len(args) > 0 else kwargs["input"]
    weight = args[1] if len(args) > 1 else kwargs["weight"]
    bias = args[2] if len(args) > 2 else kwargs.get("bias")
    out = linear_nf4(inp, weight)
    return out if bias is None else out + bias


# ---- public functions ---------------------------------------------------------------------------------
def to_nf4(tensor: torch.Tensor, block_size: Optional[int] = 64, scaler_block_size: Optional[int] = 256) -> NF4Tensor:
    """Quantise ``tensor`` to NF4 with double-quantised block scalers.

    ``None`` for either granularity selects its default (the model builders forward ``None`` when the user
    gave nothing: ``torchtune/models/llama3/_component_builders.py:177``).
    """
    if block_size is None:
        block_size = DEFAULT_BLOCK_SIZE
    if scaler_block_size is None:
        scaler_block_size = DEFAULT_SCALER_BLOCK_SIZE
    return NF4Tensor.from_tensor(tensor, block_size, scaler_block_size)


class _LinearNF4(torch.autograd.Function):
    """y = x @ D(W)^T; only the packed weight is kept for backward; no gradient for the weight."""

    @staticmethod
    def forward(ctx, input: torch.Tensor, weight: NF4Tensor):
        _check_in_features(input, weight)
        ctx.save_for_backward(weight)
        ctx.in_shape = input.shape
        if _fused_ok(input, weight, 0):
            x2 = input.reshape(-1, input.shape[-1])
            tr = weight.backward_copy_for(x2.shape[0], True)
            y = ops.nf4_lora_linear_fwd(x2, weight.quantized_data, weight.block_scalers(), weight.shape[0],
                                        block_scalers_t=tr[1] if tr else None)
            return y.view(*input.shape[:-1], weight.shape[0])
        return F.linear(input, weight.to(input.dtype))

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        (weight,) = ctx.saved_tensors
        if not ctx.needs_input_grad[0]:
            return None, None
        if _fused_ok(grad_output, weight, 0):
            g2 = grad_output.reshape(-1, grad_output.shape[-1])
            gx = ops.nf4_linear_bwd_dx(g2, weight.quantized_data, weight.block_scalers(), weight.shape[1],
                                       transposed=weight.backward_copy_for(g2.shape[0], False))
            return gx.view(ctx.in_shape), None
        return grad_output @ weight.to(grad_output.dtype), None


def _check_in_features(x: torch.Tensor, weight: torch.Tensor) -> None:
    """The shape error ``F.linear`` raises for a dense weight; the fused kernels take K from the activation, so a wrong
    inner dimension must be stopped on the host."""
    if isinstance(weight, NF4Tensor):
        shape = shape_and_dtype(weight)[0]
        if len(shape) == 2 and x.dim() > 0 and x.shape[-1] == shape[1]:
            return
    if weight.dim() == 2 and (x.dim() == 0 or x.shape[-1] != weight.shape[1]):
        raise RuntimeError(
            f"mat1 and mat2 shapes cannot be multiplied ({x.numel() // max(x.shape[-1] if x.dim() else 1, 1)}x"
            f"{x.shape[-1] if x.dim() else 1} and {weight.shape[1]}x{weight.shape[0]})"
        )


def _fused_ok(x: torch.Tensor, weight: NF4Tensor, rank: int) -> bool:
    """True when the fused dequantise-in-GEMM kernel applies; otherwise the caller dequantises with the
    stand-alone kernel and uses a library GEMM."""
    shape, dtype = shape_and_dtype(weight)
    return (
        x.is_cuda
        and weight.quantized_data.is_cuda
        and x.dtype == torch.bfloat16
        and dtype == torch.bfloat16
        and len(shape) == 2
        and weight.block_size == 64
        and x.numel() > 0
        and ops.fused_shape_ok(shape[0], shape[1], rank)
    )


def linear_nf4(input: torch.Tensor, weight: NF4Tensor) -> torch.Tensor:
    """Linear layer over a frozen NF4 weight: differentiable w.r.t. ``input`` only."""
    return _LinearNF4.apply(input, weight)
