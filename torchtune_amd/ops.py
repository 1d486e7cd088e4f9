"""Tensor-level wrappers over the C ABI: validate, allocate outputs, pass raw device pointers and the
caller's current HIP stream.  PyTorch is used here for device memory and streams only.

Every function requires HIP (``cuda``) tensors.  There is no CPU implementation in this package.
"""
from __future__ import annotations

import ctypes
import weakref
from typing import List, Optional, Sequence, Tuple

import torch

from . import _lib

_DTYPE_CODE = {torch.bfloat16: _lib.TTAMD_BF16, torch.float32: _lib.TTAMD_F32}


def _code(dtype: torch.dtype, what: str) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise TypeError(f"{what}: dtype {dtype} is not supported (bfloat16 and float32 are)") from None


def _need_gpu(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            f"{what}: expected a tensor on an AMD GPU (device 'cuda'), got device '{t.device}'. "
            "torchtune_amd computes only through its HIP kernels."
        )


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def _on_device(device: torch.device):
    """Context in which ``device`` is the current GPU: nothing to do (and nothing to pay) when it already is."""
    return _NO_GUARD if torch.cuda.current_device() == device.index else torch.cuda.device(device)


def _workspace(nbytes: int, device: torch.device) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=device)


# ---------------------------------------------------------------------------------------------------
# NF4 codec
# ---------------------------------------------------------------------------------------------------
def nf4_quantize(w: torch.Tensor, block_size: int, scaler_block_size: int):
    """-> (quantized_data u8 [numel/2], quantized_scalers i8 [n_blocks], quantization_factor dtype [n_sb],
    scaler_mean dtype 0-dim)"""
    _need_gpu(w, "nf4_quantize")
    code = _code(w.dtype, "nf4_quantize")
    w = w.detach().contiguous()
    numel = w.numel()
    if block_size <= 0 or numel % block_size != 0:
        raise ValueError(f"nf4_quantize: numel ({numel}) must be divisible by block_size ({block_size})")
    n_blocks = numel // block_size
    if scaler_block_size <= 0 or n_blocks % scaler_block_size != 0:
        raise ValueError(
            f"nf4_quantize: number of blocks ({n_blocks}) must be divisible by scaler_block_size ({scaler_block_size})"
        )
    lib = _lib.load()
    dev = w.device
    qdata = torch.empty(numel // 2, dtype=torch.uint8, device=dev)
    qscalers = torch.empty(n_blocks, dtype=torch.int8, device=dev)
    qfactor = torch.empty(n_blocks // scaler_block_size, dtype=w.dtype, device=dev)
    mean = torch.empty((), dtype=w.dtype, device=dev)
    ws_bytes = lib.ttamd_nf4_quantize_workspace_bytes(numel, block_size)
    ws = _workspace(ws_bytes, dev)
    with torch.cuda.device(dev):
        rc = lib.ttamd_nf4_quantize(
            w.data_ptr(), code, numel, block_size, scaler_block_size, qdata.data_ptr(), qscalers.data_ptr(),
            qfactor.data_ptr(), mean.data_ptr(), ws.data_ptr(), ws.numel(), _stream(w),
        )
    _lib.check(rc, "nf4_quantize")
    return qdata, qscalers, qfactor, mean


def nf4_dequantize(
    qdata: torch.Tensor, qscalers: torch.Tensor, qfactor: torch.Tensor, mean: torch.Tensor, shape, block_size: int,
    scaler_block_size: int, out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Dense weight of an NF4 tensor.  ``out`` may be a contiguous tensor on the same GPU or in pinned host memory;
    the kernel then stores straight into it (over PCIe for host memory: the caller synchronises the stream before
    reading it on the CPU)."""
    _need_gpu(qdata, "nf4_dequantize")
    dtype = qfactor.dtype
    code = _code(dtype, "nf4_dequantize")
    numel = qdata.numel() * 2
    if out is None:
        out = torch.empty(numel, dtype=dtype, device=qdata.device)
    else:
        on_device = out.is_cuda and out.device == qdata.device
        if not (on_device or (out.device.type == "cpu" and out.is_pinned())):
            raise ValueError("nf4_dequantize: `out` must live on the weight's GPU or in pinned host memory")
        if out.dtype != dtype or out.numel() != numel or not out.is_contiguous():
            raise ValueError(f"nf4_dequantize: `out` must be a contiguous {dtype} tensor of {numel} elements")
    lib = _lib.load()
    with torch.cuda.device(qdata.device):
        rc = lib.ttamd_nf4_dequantize(
            qdata.data_ptr(), qscalers.data_ptr(), qfactor.data_ptr(), mean.data_ptr(), code, numel, block_size,
            scaler_block_size, out.data_ptr(), _stream(qdata),
        )
    _lib.check(rc, "nf4_dequantize")
    return out.view(shape)


def nf4_dequantize_merge(qdata: torch.Tensor, block_scalers: torch.Tensor, N: int, K: int, lora_a: torch.Tensor,
                         lora_b: torch.Tensor, scale: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """bf16(D(W) + bf16(scale * bf16(lora_b @ lora_a))) for an NF4 [N, K] weight (block size 64) in one pass.
    ``out`` may be a contiguous bf16 [N, K] tensor on the same GPU or in pinned host memory (the kernel then stores over
    PCIe; the caller synchronises the stream before reading it on the CPU)."""
    _need_gpu(qdata, "nf4_dequantize_merge")
    a = _bf16_2d(lora_a, "nf4_dequantize_merge: lora_a")
    b = _bf16_2d(lora_b, "nf4_dequantize_merge: lora_b")
    rank = a.shape[0]
    if a.shape != (rank, K) or b.shape != (N, rank):
        raise ValueError(f"nf4_dequantize_merge: lora_a {tuple(a.shape)} / lora_b {tuple(b.shape)} do not fit [{N}, {K}]")
    if out is None:
        out = torch.empty(N, K, dtype=torch.bfloat16, device=qdata.device)
    else:
        on_device = out.is_cuda and out.device == qdata.device
        if not (on_device or (out.device.type == "cpu" and out.is_pinned())):
            raise ValueError("nf4_dequantize_merge: `out` must live on the weight's GPU or in pinned host memory")
        if out.dtype != torch.bfloat16 or tuple(out.shape) != (N, K) or not out.is_contiguous():
            raise ValueError(f"nf4_dequantize_merge: `out` must be a contiguous bfloat16 [{N}, {K}] tensor")
    lib = _lib.load()
    with torch.cuda.device(qdata.device):
        rc = lib.ttamd_nf4_dequantize_merge_bf16(qdata.data_ptr(), block_scalers.data_ptr(), a.data_ptr(), b.data_ptr(), rank,
                                                 float(scale), out.data_ptr(), N, K, _stream(qdata))
    _lib.check(rc, "nf4_dequantize_merge")
    return out


def nf4_block_scalers(qscalers: torch.Tensor, qfactor: torch.Tensor, mean: torch.Tensor, scaler_block_size: int) -> torch.Tensor:
    _need_gpu(qscalers, "nf4_block_scalers")
    code = _code(qfactor.dtype, "nf4_block_scalers")
    out = torch.empty(qscalers.numel(), dtype=torch.float32, device=qscalers.device)
    lib = _lib.load()
    with torch.cuda.device(qscalers.device):
        rc = lib.ttamd_nf4_block_scalers(
            qscalers.data_ptr(), qfactor.data_ptr(), mean.data_ptr(), code, qscalers.numel(), scaler_block_size,
            out.data_ptr(), _stream(qscalers),
        )
    _lib.check(rc, "nf4_block_scalers")
    return out


# ---------------------------------------------------------------------------------------------------
# fused NF4 + LoRA linear
# ---------------------------------------------------------------------------------------------------
_gemm_timer = None


def gemm_timer_installed() -> bool:
    """True while ``set_gemm_timer`` has a callback in place."""
    return _gemm_timer is not None


def set_gemm_timer(timer) -> None:
    """Install (or with None remove) a callback ``timer(kind, M, N, K, rank, on_tiles=False) -> (start_event, end_event)``;
    the two events are recorded on the launch stream immediately before and after every fused-GEMM launch (``kind`` "fwd" /
    "bwd"; for the group calls "fwd_group" / "bwd_group" with ``N`` and ``rank`` lists over the members; ``on_tiles``: a
    grad-input that reads the expanded weight its layer's forward call kept).  Used by the benchmark to time the
    dominant kernel in place."""
    global _gemm_timer
    _gemm_timer = timer


def fused_shape_ok(N: int, K: int, rank: int) -> bool:
    """Shapes the fused bf16 GEMM accepts (NF4 block_size must also be 64)."""
    return K % 64 == 0 and N % 64 == 0 and rank % 8 == 0 and 0 <= rank <= 64


def _bf16_2d(t: torch.Tensor, what: str) -> torch.Tensor:
    _need_gpu(t, what)
    if t.dtype != torch.bfloat16 or t.dim() != 2:
        raise TypeError(f"{what}: expected a 2-D bfloat16 tensor, got {tuple(t.shape)} {t.dtype}")
    return t.contiguous()


def _check_nf4_operands(what: str, N: int, K: int, qdata: torch.Tensor, block_scalers: torch.Tensor,
                        block_scalers_t: Optional[torch.Tensor] = None) -> None:
    """The kernels take sizes from the activation and the caller's N; the packed tensors must really hold an [N, K]
    weight (the C side sees only pointers)."""
    _need_gpu(qdata, what)
    if qdata.dtype != torch.uint8 or qdata.numel() * 2 != N * K:
        raise ValueError(f"{what}: quantized_data holds {qdata.numel() * 2} codes ({qdata.dtype}), the weight is [{N}, {K}]")
    if block_scalers.dtype != torch.float32 or block_scalers.numel() * 64 != N * K:
        raise ValueError(f"{what}: block_scalers must be float32 with {N * K // 64} elements, got {block_scalers.numel()} "
                         f"{block_scalers.dtype}")
    if block_scalers_t is not None and (block_scalers_t.dtype != torch.float32 or block_scalers_t.numel() * 64 != N * K):
        raise ValueError(f"{what}: block_scalers_t must be float32 with {N * K // 64} elements")


def _check_adapter(what: str, M: int, n_out: int, act: torch.Tensor, weight: torch.Tensor, weight_shape) -> None:
    rank = act.shape[1]
    if act.shape[0] != M:
        raise ValueError(f"{what}: the adapter activation has {act.shape[0]} rows, the input {M}")
    if tuple(weight.shape) != tuple(weight_shape(rank)):
        raise ValueError(f"{what}: the adapter weight is {tuple(weight.shape)}, expected {tuple(weight_shape(rank))}")


def lora_hidden(x: torch.Tensor, lora_a: torch.Tensor) -> torch.Tensor:
    """h = bf16(x @ lora_a.T);  x [M,K], lora_a [r,K] -> [M,r]"""
    x = _bf16_2d(x, "lora_hidden")
    lora_a = _bf16_2d(lora_a, "lora_hidden")
    M, K = x.shape
    r = lora_a.shape[0]
    if lora_a.shape[1] != K:
        raise ValueError(f"lora_hidden: x has {K} columns, lora_a {lora_a.shape[1]}")
    lib = _lib.load()
    h = torch.empty(M, r, dtype=torch.bfloat16, device=x.device)
    ws = _workspace(lib.ttamd_lora_fwd_workspace_bytes(M, K, r), x.device)
    with torch.cuda.device(x.device):
        rc = lib.ttamd_lora_hidden_bf16(x.data_ptr(), lora_a.data_ptr(), h.data_ptr(), M, K, r, ws.data_ptr(), ws.numel(),
                                        _stream(x))
    _lib.check(rc, "lora_hidden")
    return h


# Many tokens: let the library expand the NF4 weight once per call into scratch memory (2 bytes per weight element,
# freed after the call) and run its plain bf16 GEMM on it.  False keeps the fused kernel, which needs no scratch.
EXPANDED_WEIGHT_PATH = True


# One expansion for both directions: a forward call that expanded its weight hands the scratch copy to the backward of the
# same layer, whose grad-input GEMM reads those forward tiles (transposing LDS reads) instead of expanding the weight a
# second time.  The launch on forward tiles takes as long as the one on transposed tiles (within 2 % either way at 8192
# tokens), so what decides is memory: kept tiles hold 2 bytes per weight element from a layer's forward to its backward -
# every layer's at once without activation checkpointing (13 GiB for an 8B model), one layer's at a time with it (from
# the recomputation to the backward).  Measured up to 8192 tokens per call (8B step -0.8 %, 1B -1.2 % against a limit of
# 4096); 0: never keep, a large number: always.
KEEP_FORWARD_TILES_MAX_TOKENS = 8192


def keeps_forward_tiles(M: int) -> bool:
    return bool(EXPANDED_WEIGHT_PATH and 0 < M <= KEEP_FORWARD_TILES_MAX_TOKENS)


# Expanded weights kept ACROSS calls.  The base weight of a QLoRA run never changes, so the tiles a many-token forward
# expands it into can stay: every later forward and grad-input of the layer (or group of layers) then runs its GEMM on
# them and no expansion launch is left in the step.  The price is 2 bytes per weight element of device memory for as long
# as the weight lives (14 GB for an 8B model, 137 GB for a 70B one), which is why it is off unless a budget is given:
# tiles are admitted first come, first served while their sum stays within RESIDENT_TILES_MAX_BYTES, layers beyond
# the budget keep expanding per call.  The cache entries ride on the weight and are keyed like its block scalers (a write
# into the weight drops them).  Results are the same bits either way: the same tiles feed the same GEMM launch.
RESIDENT_TILES_MAX_BYTES = 0
_resident_tiles_bytes = 0


def resident_tiles_enabled() -> bool:
    return bool(EXPANDED_WEIGHT_PATH and RESIDENT_TILES_MAX_BYTES > 0)


def resident_tiles_bytes() -> int:
    """Bytes of expanded weights currently held across calls."""
    return _resident_tiles_bytes


def _resident_release(nbytes: int) -> None:
    global _resident_tiles_bytes
    _resident_tiles_bytes -= nbytes


def resident_tiles_admit(tiles: torch.Tensor) -> bool:
    """Counts ``tiles`` (a forward call's scratch memory whose head holds expanded weights) against the budget; True when
    the caller may keep it.  The bytes are given back when the tensor is freed."""
    global _resident_tiles_bytes
    nbytes = tiles.numel() * tiles.element_size()
    if not resident_tiles_enabled() or _resident_tiles_bytes + nbytes > RESIDENT_TILES_MAX_BYTES:
        return False
    _resident_tiles_bytes += nbytes
    weakref.finalize(tiles, _resident_release, nbytes)
    return True


def gemm_expands_weight(M: int, n_out: int, k_contract: int) -> bool:
    """True when an NF4 GEMM call of this shape runs on the weight expanded once per call (needs no transposed copy)."""
    return bool(EXPANDED_WEIGHT_PATH and _lib.load().ttamd_nf4_gemm_expands_weight(M, n_out, k_contract))


def _gemm_workspace(lib, M: int, n_out: int, k_contract: int, device):
    """Scratch memory for one NF4 GEMM: fp32 slices of the contraction for a launch of few output tiles, or room for the
    expanded weight of a many-token launch (None: not needed, or the expanded path is switched off)."""
    nbytes = int(lib.ttamd_nf4_gemm_workspace_bytes(M, n_out, k_contract))
    if nbytes == 0 or (not EXPANDED_WEIGHT_PATH and lib.ttamd_nf4_gemm_expands_weight(M, n_out, k_contract)):
        return None, 0
    return torch.empty(nbytes // 4, dtype=torch.float32, device=device), nbytes


def nf4_lora_linear_fwd(
    x: torch.Tensor, qdata: torch.Tensor, block_scalers: torch.Tensor, N: int, h: Optional[torch.Tensor] = None,
    lora_b: Optional[torch.Tensor] = None, scale: float = 0.0, bias: Optional[torch.Tensor] = None,
    block_scalers_t: Optional[torch.Tensor] = None, col_scale: Optional[torch.Tensor] = None, return_tiles: bool = False,
):
    """y = x @ D(W).T (+bias) + scale * h @ lora_b.T ;  x [M,K] -> [M,N].  ``block_scalers_t``: the scalers transposed
    ([K/64, N] fp32, second tensor of ``nf4_transpose_for_backward``): same result, cheaper scaler loads.

    ``return_tiles=True`` returns ``(y, tiles)``: the call's scratch memory when it holds the weight expanded in forward
    tile order (many tokens; what ``tiled_linear_dx`` reads), else ``None``."""
    x = _bf16_2d(x, "nf4_lora_linear_fwd")
    M, K = x.shape
    _check_nf4_operands("nf4_lora_linear_fwd", N, K, qdata, block_scalers, block_scalers_t)
    rank = 0
    if h is not None:
        h = _bf16_2d(h, "nf4_lora_linear_fwd")
        lora_b = _bf16_2d(lora_b, "nf4_lora_linear_fwd")
        rank = h.shape[1]
        _check_adapter("nf4_lora_linear_fwd", M, N, h, lora_b, lambda r: (N, r))
    if bias is not None:
        bias = bias.contiguous()
        if bias.dtype != torch.bfloat16:
            raise TypeError("nf4_lora_linear_fwd: bias must be bfloat16")
        if bias.numel() != N:
            raise ValueError(f"nf4_lora_linear_fwd: bias has {bias.numel()} elements, the layer {N} outputs")
    if col_scale is not None and col_scale.numel() != N:
        raise ValueError(f"nf4_lora_linear_fwd: col_scale has {col_scale.numel()} elements, the layer {N} outputs")
    y = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
    lib = _lib.load()
    ws, ws_bytes = _gemm_workspace(lib, M, N, K, x.device)
    with torch.cuda.device(x.device):
        events = _gemm_timer("fwd", M, N, K, rank) if _gemm_timer is not None else None
        if events:
            events[0].record()
        if col_scale is not None:  # DoRA: every output column times magnitude / weight norm
            col_scale = _bf16_any(col_scale, "nf4_lora_linear_fwd: col_scale")
        rc = lib.ttamd_nf4_lora_linear_fwd_ws_bf16(
            x.data_ptr(), qdata.data_ptr(), block_scalers.data_ptr(), _ptr(block_scalers_t), _ptr(h), _ptr(lora_b), rank,
            float(scale), _ptr(bias), _ptr(col_scale), y.data_ptr(), M, N, K, _ptr(ws), ws_bytes, _stream(x),
        )
        if events:
            events[1].record()
    _lib.check(rc, "nf4_lora_linear_fwd")
    if return_tiles:
        return y, (ws if ws is not None and lib.ttamd_nf4_gemm_expands_weight(M, N, K) else None)
    return y


def nf4_transpose_for_backward(qdata: torch.Tensor, block_scalers: torch.Tensor, N: int, K: int):
    """-> (codes re-packed along N: u8 [K*N/2], block scalers transposed: fp32 [K/64, N])"""
    _check_nf4_operands("nf4_transpose_for_backward", N, K, qdata, block_scalers)
    qdata_t = torch.empty(K * N // 2, dtype=torch.uint8, device=qdata.device)
    scal_t = torch.empty(K // 64, N, dtype=torch.float32, device=qdata.device)
    lib = _lib.load()
    with torch.cuda.device(qdata.device):
        rc = lib.ttamd_nf4_transpose_for_backward(qdata.data_ptr(), block_scalers.data_ptr(), N, K, qdata_t.data_ptr(),
                                                  scal_t.data_ptr(), _stream(qdata))
    _lib.check(rc, "nf4_transpose_for_backward")
    return qdata_t, scal_t


def nf4_linear_bwd_dx(
    gy: torch.Tensor, qdata: torch.Tensor, block_scalers: torch.Tensor, K: int, gh: Optional[torch.Tensor] = None,
    lora_a: Optional[torch.Tensor] = None, transposed=None, swiglu: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
):
    """gx = gy @ D(W) + gh @ lora_a ;  gy [M,N] -> [M,K].  `transposed` = the pair from nf4_transpose_for_backward
    (fast path) or None (the weight tile is transposed on the fly).

    ``swiglu=(gate, up)`` ([M,K] each): gx is the gradient of ``silu(gate) * up``; the call returns
    ``(ggate, gup) = swiglu_bwd(gx, gate, up)`` (the same bits) instead of gx, from the GEMM's own epilogue on the
    many-token path."""
    gy = _bf16_2d(gy, "nf4_linear_bwd_dx")
    M, N = gy.shape
    _check_nf4_operands("nf4_linear_bwd_dx", N, K, qdata, block_scalers, transposed[1] if transposed else None)
    if transposed and (transposed[0].dtype != torch.uint8 or transposed[0].numel() * 2 != N * K):
        raise ValueError(f"nf4_linear_bwd_dx: the transposed codes do not hold a [{N}, {K}] weight")
    rank = 0
    if gh is not None:
        gh = _bf16_2d(gh, "nf4_linear_bwd_dx")
        lora_a = _bf16_2d(lora_a, "nf4_linear_bwd_dx")
        rank = gh.shape[1]
        _check_adapter("nf4_linear_bwd_dx", M, K, gh, lora_a, lambda r: (r, K))
    gx = torch.empty(M, K, dtype=torch.bfloat16, device=gy.device)
    gup = None
    if swiglu is not None:
        gate, up = (_bf16_2d(t, "nf4_linear_bwd_dx") for t in swiglu)
        if tuple(gate.shape) != (M, K) or tuple(up.shape) != (M, K):
            raise ValueError(f"nf4_linear_bwd_dx: gate {tuple(gate.shape)} and up {tuple(up.shape)} must both be [{M}, {K}]")
        gup = torch.empty_like(gx)
    lib = _lib.load()
    # without the transposed copy only the expanded-weight path takes a workspace (the first-generation kernel slices nothing)
    ws, ws_bytes = _gemm_workspace(lib, M, K, N, gy.device) if transposed or lib.ttamd_nf4_gemm_expands_weight(M, K, N) else (None, 0)
    with torch.cuda.device(gy.device):
        events = _gemm_timer("bwd" if swiglu is None else "bwd_swiglu", M, N, K, rank) if _gemm_timer is not None else None
        if events:
            events[0].record()
        head = (gy.data_ptr(), qdata.data_ptr(), block_scalers.data_ptr(), _ptr(transposed[0]) if transposed else None,
                _ptr(transposed[1]) if transposed else None, _ptr(gh), _ptr(lora_a), rank)
        if swiglu is None:
            rc = lib.ttamd_nf4_linear_bwd_dx_ws_bf16(*head, gx.data_ptr(), M, N, K, _ptr(ws), ws_bytes, _stream(gy))
        else:
            rc = lib.ttamd_nf4_linear_bwd_dx_swiglu_ws_bf16(*head, gate.data_ptr(), up.data_ptr(), gx.data_ptr(), gup.data_ptr(),
                                                            M, N, K, _ptr(ws), ws_bytes, _stream(gy))
        if events:
            events[1].record()
    _lib.check(rc, "nf4_linear_bwd_dx")
    return gx if swiglu is None else (gx, gup)


def lora_bwd(
    gy: torch.Tensor, x: torch.Tensor, h: torch.Tensor, lora_b: torch.Tensor, scale: float
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """-> (gh [M,r], gA [r,K], gB [N,r])"""
    gy = _bf16_2d(gy, "lora_bwd")
    x = _bf16_2d(x, "lora_bwd")
    h = _bf16_2d(h, "lora_bwd")
    lora_b = _bf16_2d(lora_b, "lora_bwd")
    M, N = gy.shape
    K = x.shape[1]
    r = h.shape[1]
    if x.shape[0] != M or h.shape[0] != M or tuple(lora_b.shape) != (N, r):
        raise ValueError(f"lora_bwd: gy {tuple(gy.shape)}, x {tuple(x.shape)}, h {tuple(h.shape)} and lora_b "
                         f"{tuple(lora_b.shape)} do not belong to one layer")
    dev = gy.device
    gh = torch.empty(M, r, dtype=torch.bfloat16, device=dev)
    ga = torch.empty(r, K, dtype=torch.bfloat16, device=dev)
    gb = torch.empty(N, r, dtype=torch.bfloat16, device=dev)
    lib = _lib.load()
    ws = _workspace(lib.ttamd_lora_bwd_workspace_bytes(M, N, K, r), dev)
    with torch.cuda.device(dev):
        rc = lib.ttamd_lora_bwd_bf16(
            gy.data_ptr(), x.data_ptr(), h.data_ptr(), lora_b.data_ptr(), float(scale), gh.data_ptr(), ga.data_ptr(),
            gb.data_ptr(), M, N, K, r, ws.data_ptr(), ws.numel(), _stream(gy),
        )
    _lib.check(rc, "lora_bwd")
    return gh, ga, gb


# ---------------------------------------------------------------------------------------------------
# The whole layer, one library call per direction
# ---------------------------------------------------------------------------------------------------
def qlora_linear_fwd(
    x: torch.Tensor, qdata: torch.Tensor, block_scalers: torch.Tensor, N: int, lora_a: torch.Tensor, lora_b: torch.Tensor,
    scale: float, bias: Optional[torch.Tensor] = None, block_scalers_t: Optional[torch.Tensor] = None, return_tiles: bool = False,
):
    """``(y, h)``: ``h = bf16(x @ lora_a.T)`` and ``y = x @ D(W).T (+ bias) + scale * h @ lora_b.T`` from one call of
    ``ttamd_qlora_linear_fwd_bf16`` (``lora_hidden`` followed by ``nf4_lora_linear_fwd``, the same launches and bits, out
    of one workspace).  ``return_tiles=True``: ``(y, h, tiles)`` with the call's workspace when its head holds the weight
    expanded in forward tile order (many tokens), else ``None``."""
    x = _bf16_2d(x, "qlora_linear_fwd")
    lora_a = _bf16_2d(lora_a, "qlora_linear_fwd")
    lora_b = _bf16_2d(lora_b, "qlora_linear_fwd")
    M, K = x.shape
    rank = lora_a.shape[0]
    _check_nf4_operands("qlora_linear_fwd", N, K, qdata, block_scalers, block_scalers_t)
    if lora_a.shape[1] != K or tuple(lora_b.shape) != (N, rank):
        raise ValueError(f"qlora_linear_fwd: lora_a {tuple(lora_a.shape)} / lora_b {tuple(lora_b.shape)} do not fit a "
                         f"[{N}, {K}] layer")
    if bias is not None:
        bias = bias.contiguous()
        if bias.dtype != torch.bfloat16 or bias.numel() != N:
            raise ValueError(f"qlora_linear_fwd: bias must be bfloat16 with {N} elements")
    lib = _lib.load()
    y = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
    h = torch.empty(M, rank, dtype=torch.bfloat16, device=x.device)
    nbytes = int(lib.ttamd_qlora_linear_fwd_workspace_bytes(M, N, K, rank))
    ws = _workspace(nbytes, x.device)
    with _on_device(x.device):
        rc = lib.ttamd_qlora_linear_fwd_bf16(
            x.data_ptr(), qdata.data_ptr(), block_scalers.data_ptr(), _ptr(block_scalers_t), lora_a.data_ptr(), lora_b.data_ptr(),
            rank, float(scale), _ptr(bias), y.data_ptr(), h.data_ptr(), M, N, K, ws.data_ptr(), ws.numel(), _stream(x))
    _lib.check(rc, "qlora_linear_fwd")
    if return_tiles:
        return y, h, (ws if EXPANDED_WEIGHT_PATH and lib.ttamd_nf4_gemm_expands_weight(M, N, K) else None)
    return y, h


def qlora_linear_bwd(
    gy: torch.Tensor, x: torch.Tensor, h: torch.Tensor, qdata: torch.Tensor, block_scalers: torch.Tensor, lora_a: torch.Tensor,
    lora_b: torch.Tensor, scale: float, transposed=None, need_gx: bool = True, tiles: Optional[torch.Tensor] = None,
) -> Tuple[Optional[torch.Tensor], torch.Tensor, torch.Tensor]:
    """``(gx or None, gA, gB)`` from one call of ``ttamd_qlora_linear_bwd_bf16`` (``lora_bwd`` followed by
    ``nf4_linear_bwd_dx``, the same launches and bits, out of one workspace that also holds ``gh``).  ``tiles``: the
    forward call's expanded weight (``qlora_linear_fwd(..., return_tiles=True)``); the grad-input then reads it instead
    of expanding the weight again."""
    gy = _bf16_2d(gy, "qlora_linear_bwd")
    x = _bf16_2d(x, "qlora_linear_bwd")
    h = _bf16_2d(h, "qlora_linear_bwd")
    lora_a = _bf16_2d(lora_a, "qlora_linear_bwd")
    lora_b = _bf16_2d(lora_b, "qlora_linear_bwd")
    M, N = gy.shape
    K = x.shape[1]
    rank = h.shape[1]
    _check_nf4_operands("qlora_linear_bwd", N, K, qdata, block_scalers, transposed[1] if transposed else None)
    if transposed and (transposed[0].dtype != torch.uint8 or transposed[0].numel() * 2 != N * K):
        raise ValueError(f"qlora_linear_bwd: the transposed codes do not hold a [{N}, {K}] weight")
    if x.shape[0] != M or h.shape[0] != M or tuple(lora_b.shape) != (N, rank) or tuple(lora_a.shape) != (rank, K):
        raise ValueError(f"qlora_linear_bwd: gy {tuple(gy.shape)}, x {tuple(x.shape)}, h {tuple(h.shape)}, lora_a "
                         f"{tuple(lora_a.shape)} and lora_b {tuple(lora_b.shape)} do not belong to one layer")
    dev = gy.device
    lib = _lib.load()
    gx = torch.empty(M, K, dtype=torch.bfloat16, device=dev) if need_gx else None
    ga = torch.empty(rank, K, dtype=torch.bfloat16, device=dev)
    gb = torch.empty(N, rank, dtype=torch.bfloat16, device=dev)
    if tiles is not None and (tiles.numel() * tiles.element_size() < 2 * N * K or not tiles.is_contiguous()):
        raise ValueError(f"qlora_linear_bwd: the forward tiles must be contiguous and hold {N} x {K} bfloat16 elements")
    if tiles is not None or not need_gx:  # no scratch memory for the GEMM stage
        nbytes = ((M * rank * 2 + 255) // 256 + (int(lib.ttamd_lora_bwd_workspace_bytes(M, N, K, rank)) + 255) // 256) * 256
    else:
        nbytes = int(lib.ttamd_qlora_linear_bwd_workspace_bytes(M, N, K, rank))
    ws = _workspace(nbytes, dev)
    with _on_device(dev):
        rc = lib.ttamd_qlora_linear_bwd_bf16(
            gy.data_ptr(), x.data_ptr(), h.data_ptr(), qdata.data_ptr(), block_scalers.data_ptr(),
            _ptr(transposed[0]) if transposed else None, _ptr(transposed[1]) if transposed else None,
            _ptr(tiles) if need_gx else None, lora_a.data_ptr(), lora_b.data_ptr(), rank, float(scale), _ptr(gx), ga.data_ptr(),
            gb.data_ptr(), M, N, K, ws.data_ptr(), ws.numel(), _stream(gy))
    _lib.check(rc, "qlora_linear_bwd")
    return gx, ga, gb


# ---------------------------------------------------------------------------------------------------
# Groups of LoRA linears with a common input (q/k/v, gate/up)
# ---------------------------------------------------------------------------------------------------
class GroupMember:
    """Operands of one member: the NF4 parts of its [N, K] weight, its adapter, its bias (or None) and alpha / rank.
    ``transposed`` is the pair from ``nf4_transpose_for_backward`` or None."""

    __slots__ = ("qdata", "block_scalers", "transposed", "lora_a", "lora_b", "bias", "scale", "N")

    def __init__(self, qdata, block_scalers, transposed, lora_a, lora_b, bias, scale: float, N: int):
        self.qdata, self.block_scalers, self.transposed = qdata, block_scalers, transposed
        self.lora_a, self.lora_b, self.bias, self.scale, self.N = lora_a, lora_b, bias, float(scale), int(N)


def group_shape_ok(Ns: Sequence[int], K: int, ranks: Sequence[int]) -> bool:
    """Shapes the group entry points accept."""
    return (1 <= len(Ns) <= _lib.GROUP_MAX and K % 64 == 0 and all(n % 64 == 0 for n in Ns)
            and all(r > 0 and r % 8 == 0 for r in ranks) and sum(ranks) <= 64 and max(Ns) >= 128)


def group_dx_expands(M: int, K: int, Ns: Sequence[int]) -> bool:
    """True when the grouped grad-input of these members runs on the expanded-weight path, which needs no transposed copies."""
    return bool(EXPANDED_WEIGHT_PATH and all(n % 64 == 0 for n in Ns) and _lib.load().ttamd_nf4_gemm_expands_weight(M, K, sum(Ns)))


def _group_array(what: str, members: Sequence[GroupMember], K: int, ys: Sequence[torch.Tensor], M: int,
                 grads: Optional[Sequence[Tuple[torch.Tensor, torch.Tensor]]] = None):
    """The C array of member descriptors (and the tensors it points into, which the caller keeps alive)."""
    if not 1 <= len(members) <= _lib.GROUP_MAX:
        raise ValueError(f"{what}: a group has 1 to {_lib.GROUP_MAX} members, got {len(members)}")
    arr = (_lib.LoraGroupMember * len(members))()
    keep = []
    for i, m in enumerate(members):
        _check_nf4_operands(what, m.N, K, m.qdata, m.block_scalers, m.transposed[1] if m.transposed else None)
        if m.transposed and (m.transposed[0].dtype != torch.uint8 or m.transposed[0].numel() * 2 != m.N * K):
            raise ValueError(f"{what}: the transposed codes of member {i} do not hold a [{m.N}, {K}] weight")
        a, b = _bf16_2d(m.lora_a, what), _bf16_2d(m.lora_b, what)
        r = a.shape[0]
        if tuple(a.shape) != (r, K) or tuple(b.shape) != (m.N, r):
            raise ValueError(f"{what}: member {i}: lora_a {tuple(a.shape)} / lora_b {tuple(b.shape)} do not fit a [{m.N}, {K}] layer")
        y = ys[i]
        if y.dtype != torch.bfloat16 or tuple(y.shape) != (M, m.N) or not y.is_contiguous():
            raise ValueError(f"{what}: member {i}: expected a contiguous bfloat16 [{M}, {m.N}] tensor, got {tuple(y.shape)} {y.dtype}")
        bias = None
        if m.bias is not None:
            bias = m.bias.contiguous()
            if bias.dtype != torch.bfloat16 or bias.numel() != m.N:
                raise ValueError(f"{what}: member {i}: bias must be bfloat16 with {m.N} elements")
        e = arr[i]
        e.quantized_data, e.block_scalers = m.qdata.data_ptr(), m.block_scalers.data_ptr()
        e.block_scalers_t = m.transposed[1].data_ptr() if m.transposed else None
        e.quantized_data_t = m.transposed[0].data_ptr() if m.transposed else None
        e.lora_a, e.lora_b, e.bias, e.y = a.data_ptr(), b.data_ptr(), _ptr(bias), y.data_ptr()
        if grads is not None:
            e.grad_lora_a, e.grad_lora_b = grads[i][0].data_ptr(), grads[i][1].data_ptr()
        e.N, e.rank, e.scale = m.N, r, m.scale
        keep.append((a, b, bias, y))
    return arr, keep


def lora_group_fwd(x: torch.Tensor, members: Sequence[GroupMember], swiglu: bool = False, return_tiles: bool = False,
                   tiles: Optional[torch.Tensor] = None, paired: bool = False):
    """-> (h_cat [M, sum of ranks], [y_i [M, N_i]]): every member's ``y_i = x @ D(W_i).T (+ bias_i) + scale_i * h_i @ B_i.T``
    with ``h_i = x @ A_i.T`` (columns of ``h_cat``), in one pass over ``x`` for the hidden products.

    ``swiglu=True`` (two members of equal width: gate, up) appends ``act = silu(y_0) * y_1`` to the list, formed in the
    epilogue of the GEMM launch where the many-token path serves the shape (``ttamd_nf4_lora_group_swiglu_fwd_bf16``).

    ``return_tiles=True`` appends ``(tiles, paired)`` to the result: the call's scratch memory when its head holds the
    members' weights expanded in forward tile order (``paired``: in the gated pair's layout), else ``(None, False)`` -
    what ``lora_group_bwd(..., tiles=..., paired=...)`` takes.

    ``tiles`` / ``paired``: such a pair from an earlier call with the same members (weights unchanged since) and the same
    ``swiglu``; where this call would expand the weights into the same layout it runs its GEMM on them instead
    (``ttamd_nf4_lora_group_fwd_tiles_bf16``), otherwise they are ignored."""
    x = _bf16_2d(x, "lora_group_fwd")
    M, K = x.shape
    dev = x.device
    if swiglu and (len(members) != 2 or members[0].N != members[1].N):
        raise ValueError("lora_group_fwd: swiglu takes the gate and the up projection, two members of equal width")
    ys = [torch.empty(M, m.N, dtype=torch.bfloat16, device=dev) for m in members]
    arr, keep = _group_array("lora_group_fwd", members, K, ys, M)
    n = len(members)
    r_total = sum(int(e.rank) for e in arr)
    h_cat = torch.empty(M, r_total, dtype=torch.bfloat16, device=dev)
    lib = _lib.load()
    fwd_bytes = lib.ttamd_lora_group_fwd_workspace_bytes(arr, n, M, K)
    if not EXPANDED_WEIGHT_PATH and any(lib.ttamd_nf4_gemm_expands_weight(M, m.N, K) for m in members):
        fwd_bytes = 0  # less than the library asks for: it keeps the fused kernel
    on_tiles = (tiles is not None and fwd_bytes > 0
                and int(lib.ttamd_nf4_group_fwd_leaves_tiles(arr, n, M, K, 1 if swiglu else 0)) == (2 if paired else 1))
    if on_tiles and (tiles.numel() * tiles.element_size() < 2 * K * sum(m.N for m in members) or not tiles.is_contiguous()):
        raise ValueError("lora_group_fwd: the given tiles do not hold the members' weights")
    ws = _workspace(max(lib.ttamd_lora_group_hidden_workspace_bytes(arr, n, M, K), 0 if on_tiles else fwd_bytes), dev)
    with torch.cuda.device(dev):
        rc = lib.ttamd_lora_group_hidden_bf16(x.data_ptr(), arr, n, h_cat.data_ptr(), M, K, ws.data_ptr(), ws.numel(), _stream(x))
        _lib.check(rc, "lora_group_hidden")
        events = (_gemm_timer("fwd_gated" if swiglu else "fwd_group", M, [m.N for m in members], K, [int(e.rank) for e in arr])
                  if _gemm_timer is not None else None)
        if events:
            events[0].record()
        act = torch.empty(M, members[0].N, dtype=torch.bfloat16, device=dev) if swiglu else None
        if on_tiles:
            rc = lib.ttamd_nf4_lora_group_fwd_tiles_bf16(x.data_ptr(), arr, n, h_cat.data_ptr(), _ptr(act), M, K, tiles.data_ptr(),
                                                         1 if paired else 0, _stream(x))
        elif swiglu:
            rc = lib.ttamd_nf4_lora_group_swiglu_fwd_bf16(x.data_ptr(), arr, n, h_cat.data_ptr(), act.data_ptr(), M, K, ws.data_ptr(),
                                                          ws.numel(), _stream(x))
        else:
            rc = lib.ttamd_nf4_lora_group_fwd_bf16(x.data_ptr(), arr, n, h_cat.data_ptr(), M, K, ws.data_ptr(), ws.numel(), _stream(x))
        if events:
            events[1].record()
    _lib.check(rc, "lora_group_fwd")
    outs = ys + [act] if swiglu else ys
    if return_tiles:
        del keep
        if on_tiles:
            return h_cat, outs, tiles, paired
        layout = int(lib.ttamd_nf4_group_fwd_leaves_tiles(arr, n, M, K, 1 if swiglu else 0)) if fwd_bytes else 0
        return h_cat, outs, (ws if layout else None), layout == 2
    del keep
    return h_cat, outs


def lora_group_bwd(x: torch.Tensor, h_cat: torch.Tensor, members: Sequence[GroupMember], gys: Optional[Sequence[torch.Tensor]],
                   want_gx: bool = True, tiles: Optional[torch.Tensor] = None, paired: bool = False, swiglu=None):
    """-> (gx [M, K] or None, [(gA_i, gB_i)], gh_cat): the backward of ``lora_group_fwd`` given the output gradients.
    ``tiles`` / ``paired``: what the forward call returned with ``return_tiles=True``; the grouped grad-input then reads
    those tiles instead of expanding the members' weights again.

    ``swiglu=(gact, gate, up)`` (two members of equal width, the gate and the up projection; ``gys`` None): the output
    gradients are those of ``act = silu(gate) * up`` given the gradient of ``act`` - ``swiglu_bwd(gact, gate, up)``, formed
    by the library in the pass that multiplies them with the adapters where such a pass exists
    (``ttamd_lora_group_swiglu_bwd_bf16``); same results as the two steps."""
    x = _bf16_2d(x, "lora_group_bwd")
    h_cat = _bf16_2d(h_cat, "lora_group_bwd")
    M, K = x.shape
    dev = x.device
    if swiglu is not None:
        if gys is not None or len(members) != 2 or members[0].N != members[1].N:
            raise ValueError("lora_group_bwd: swiglu takes the gate and the up projection (equal widths) and no output gradients")
        sw = [_bf16_2d(t, "lora_group_bwd") for t in swiglu]
        if any(tuple(t.shape) != (M, members[0].N) for t in sw):
            raise ValueError(f"lora_group_bwd: gact, gate and up must be [{M}, {members[0].N}]")
        gys = [torch.empty(M, members[0].N, dtype=torch.bfloat16, device=dev) for _ in range(2)]
    gys = [_bf16_2d(g, "lora_group_bwd") for g in gys]
    grads = [(torch.empty(m.lora_a.shape, dtype=torch.bfloat16, device=dev), torch.empty(m.lora_b.shape, dtype=torch.bfloat16, device=dev))
             for m in members]
    arr, keep = _group_array("lora_group_bwd", members, K, gys, M, grads)
    n = len(members)
    r_total = sum(int(e.rank) for e in arr)
    if tuple(h_cat.shape) != (M, r_total):
        raise ValueError(f"lora_group_bwd: h_cat is {tuple(h_cat.shape)}, expected {(M, r_total)}")
    if want_gx and tiles is None and any(m.transposed is None for m in members) and not (
            EXPANDED_WEIGHT_PATH and _lib.load().ttamd_nf4_group_bwd_dx_workspace_bytes(arr, len(members), M, K)):
        raise ValueError("lora_group_bwd: the grouped grad-input needs every member's transposed copy (or a shape the "
                         "expanded-weight path serves)")
    gh_cat = torch.empty(M, r_total, dtype=torch.bfloat16, device=dev)
    gx = torch.empty(M, K, dtype=torch.bfloat16, device=dev) if want_gx else None
    lib = _lib.load()
    ws = _workspace(lib.ttamd_lora_group_bwd_workspace_bytes(arr, n, M, K), dev)
    with torch.cuda.device(dev):
        if swiglu is not None:
            rc = lib.ttamd_lora_group_swiglu_bwd_bf16(x.data_ptr(), h_cat.data_ptr(), arr, n, sw[0].data_ptr(), sw[1].data_ptr(),
                                                      sw[2].data_ptr(), gh_cat.data_ptr(), M, K, ws.data_ptr(), ws.numel(), _stream(x))
        else:
            rc = lib.ttamd_lora_group_bwd_bf16(x.data_ptr(), h_cat.data_ptr(), arr, n, gh_cat.data_ptr(), M, K, ws.data_ptr(), ws.numel(),
                                               _stream(x))
        _lib.check(rc, "lora_group_bwd")
        if want_gx:
            events = (_gemm_timer("bwd_group", M, [m.N for m in members], K, [int(e.rank) for e in arr], on_tiles=tiles is not None)
                      if _gemm_timer is not None else None)
            if tiles is not None:
                if tiles.numel() * tiles.element_size() < 2 * K * sum(m.N for m in members) or not tiles.is_contiguous():
                    raise ValueError("lora_group_bwd: the forward tiles do not hold the members' weights")
                if events:
                    events[0].record()
                rc = lib.ttamd_nf4_group_bwd_dx_tiles_bf16(arr, n, gh_cat.data_ptr(), gx.data_ptr(), M, K, tiles.data_ptr(),
                                                           1 if paired else 0, _stream(x))
            else:
                dx_bytes = int(lib.ttamd_nf4_group_bwd_dx_workspace_bytes(arr, n, M, K)) if EXPANDED_WEIGHT_PATH else 0
                dx_ws = torch.empty(dx_bytes // 4, dtype=torch.float32, device=dev) if dx_bytes else None
                if events:
                    events[0].record()
                rc = lib.ttamd_nf4_group_bwd_dx_ws_bf16(arr, n, gh_cat.data_ptr(), gx.data_ptr(), M, K,
                                                        dx_ws.data_ptr() if dx_ws is not None else None, dx_bytes, _stream(x))
            if events:
                events[1].record()
            _lib.check(rc, "nf4_group_bwd_dx")
    del keep
    return gx, grads, gh_cat


# ---------------------------------------------------------------------------------------------------
# QAT fake quantisation
# ---------------------------------------------------------------------------------------------------
_fq_timer = None


def set_fq_timer(timer) -> None:
    """Install (or with None remove) a callback ``timer(kind, rows, K, group_size, elem_bytes) -> (start_event,
    end_event)``; the events are recorded on the launch stream around every fake-quant launch (``kind`` is
    ``"per_token"`` or ``"per_group"``).  Used by the benchmark to time the kernels in place."""
    global _fq_timer
    _fq_timer = timer


def _conventions(eps_per_token=None, eps_per_group_sym=None, min_scale_uint4=None, clamp_range_first=False):
    """The ``ttamd_fq_conventions`` struct for non-default constants, or None (the library's defaults: 2^-23 for both
    eps, 1e-6 for the uint4 scale, scale clamped after the division by 15)."""
    if eps_per_token is None and eps_per_group_sym is None and min_scale_uint4 is None and not clamp_range_first:
        return None
    import ctypes

    f32eps = float(torch.finfo(torch.float32).eps)
    c = _lib.FqConventions(
        f32eps if eps_per_token is None else float(eps_per_token),
        f32eps if eps_per_group_sym is None else float(eps_per_group_sym),
        1e-6 if min_scale_uint4 is None else float(min_scale_uint4),
        int(bool(clamp_range_first)),
    )
    return ctypes.byref(c)


def fq_per_token_int8_asym(x: torch.Tensor, want_qparams: bool = True, qparam_dtype: torch.dtype = torch.float32,
                           eps: Optional[float] = None):
    """x [..., K] -> (fake-quantised x, scale fp32 [rows] | None, zero_point int32 [rows] | None).
    ``qparam_dtype=torch.bfloat16`` rounds the scale to bf16 before it quantises and dequantises.
    ``eps``: lower bound of the scale (None = ``finfo(float32).eps``, the convention the oracle documents)."""
    _need_gpu(x, "fq_per_token_int8_asym")
    code = _code(x.dtype, "fq_per_token_int8_asym")
    qcode = _code(qparam_dtype, "fq_per_token_int8_asym (qparams)")
    xc = x.contiguous()
    K = xc.shape[-1]
    rows = xc.numel() // K
    out = torch.empty_like(xc)
    scale = torch.empty(rows, dtype=torch.float32, device=x.device) if want_qparams else None
    zp = torch.empty(rows, dtype=torch.int32, device=x.device) if want_qparams else None
    lib = _lib.load()
    with torch.cuda.device(x.device):
        events = _fq_timer("per_token", rows, K, 0, xc.element_size()) if _fq_timer is not None else None
        if events:
            events[0].record()
        rc = lib.ttamd_fq_per_token_int8_asym_conv(xc.data_ptr(), code, rows, K, qcode, out.data_ptr(), _ptr(scale), _ptr(zp),
                                                   _conventions(eps_per_token=eps), _stream(x))
        if events:
            events[1].record()
    _lib.check(rc, "fq_per_token_int8_asym")
    return out, scale, zp


def fq_per_group_int4_sym(w: torch.Tensor, group_size: int, want_scale: bool = True,
                          qparam_dtype: torch.dtype = torch.float32, eps: Optional[float] = None):
    """w [..., K] -> (fake-quantised w, scale fp32 [rows, K/g] | None).
    ``qparam_dtype=torch.bfloat16`` rounds the scales to bf16 before they quantise and dequantise.
    ``eps``: lower bound of the scale (None = ``finfo(float32).eps``)."""
    _need_gpu(w, "fq_per_group_int4_sym")
    code = _code(w.dtype, "fq_per_group_int4_sym")
    qcode = _code(qparam_dtype, "fq_per_group_int4_sym (qparams)")
    wc = w.contiguous()
    K = wc.shape[-1]
    rows = wc.numel() // K
    out = torch.empty_like(wc)
    scale = torch.empty(rows, K // max(group_size, 1), dtype=torch.float32, device=w.device) if want_scale else None
    lib = _lib.load()
    with torch.cuda.device(w.device):
        events = _fq_timer("per_group", rows, K, group_size, wc.element_size()) if _fq_timer is not None else None
        if events:
            events[0].record()
        rc = lib.ttamd_fq_per_group_int4_sym_conv(wc.data_ptr(), code, rows, K, group_size, qcode, out.data_ptr(), _ptr(scale),
                                                  _conventions(eps_per_group_sym=eps), _stream(w))
        if events:
            events[1].record()
    _lib.check(rc, "fq_per_group_int4_sym")
    return out, scale


def tiled_weight_shape_ok(N: int, K: int, group_size: int) -> bool:
    """Shapes ``fq_per_group_int4_sym_tiled`` / ``tiled_linear`` serve."""
    return N % 64 == 0 and K % 64 == 0 and group_size in (32, 64, 128, 256) and K % group_size == 0


def fq_per_group_int4_sym_tiled(w: torch.Tensor, group_size: int, forward: bool = True, backward: bool = True,
                                want_scale: bool = True, qparam_dtype: torch.dtype = torch.float32, eps: Optional[float] = None):
    """bf16 w [N, K] -> (fq(w) in the tiled layout ``tiled_linear`` reads for ``x @ fq(w).T`` | None, fq(w).T in that layout
    for ``gy @ fq(w)`` | None, scale fp32 [N, K/g] | None): the values of ``fq_per_group_int4_sym``, never written row-major."""
    _need_gpu(w, "fq_per_group_int4_sym_tiled")
    if w.dtype != torch.bfloat16 or w.dim() != 2:
        raise TypeError("fq_per_group_int4_sym_tiled: w must be a 2-D bfloat16 tensor")
    qcode = _code(qparam_dtype, "fq_per_group_int4_sym_tiled (qparams)")
    wc = w.contiguous()
    N, K = wc.shape
    if not tiled_weight_shape_ok(N, K, group_size):
        raise ValueError(f"fq_per_group_int4_sym_tiled: N ({N}) and K ({K}) must be multiples of 64, group_size ({group_size}) one of 32/64/128/256 dividing K")
    tf = torch.empty(N * K, dtype=torch.bfloat16, device=w.device) if forward else None
    tb = torch.empty(N * K, dtype=torch.bfloat16, device=w.device) if backward else None
    scale = torch.empty(N, K // group_size, dtype=torch.float32, device=w.device) if want_scale else None
    lib = _lib.load()
    with torch.cuda.device(w.device):
        events = _fq_timer(f"per_group_tiled{int(forward) + int(backward)}", N, K, group_size, 2) if _fq_timer is not None else None
        if events:
            events[0].record()
        rc = lib.ttamd_fq_per_group_int4_sym_tiled_bf16(wc.data_ptr(), N, K, group_size, qcode,
                                                        float(torch.finfo(torch.float32).eps) if eps is None else float(eps),
                                                        _ptr(tf), _ptr(tb), _ptr(scale), _stream(w))
        if events:
            events[1].record()
    _lib.check(rc, "fq_per_group_int4_sym_tiled")
    return tf, tb, scale


def fq_int4_sym_tiled_group(ws: Sequence[torch.Tensor], group_size: int, forward: bool = True, backward: bool = True,
                            qparam_dtype: torch.dtype = torch.float32, eps: Optional[float] = None, paired: bool = False):
    """Weights [N_i, K] of layers with a common input -> (forward tiles of the weights stacked along N | None, transposed
    tiles of the same stack | None, [scale_i fp32 [N_i, K/g]]): what ``tiled_linear_group_fwd`` / ``tiled_linear_group_dx``
    read.  Each member's values are those of ``fq_per_group_int4_sym`` on it alone.  ``paired`` (two members of equal
    shape): the forward tiles alternate 128 columns of the one with 128 of the other, what the gated group forward reads."""
    K = ws[0].shape[1]
    if paired and (len(ws) != 2 or ws[0].shape != ws[1].shape or ws[0].shape[0] % 128):
        raise ValueError("fq_int4_sym_tiled_group: the paired layout takes two weights of equal shape, N a multiple of 128")
    for w in ws:
        _need_gpu(w, "fq_int4_sym_tiled_group")
        if w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != K or not tiled_weight_shape_ok(w.shape[0], K, group_size):
            raise ValueError("fq_int4_sym_tiled_group: members must be 2-D bfloat16 weights over one K, N and K multiples of 64, "
                             f"group_size ({group_size}) one of 32/64/128/256 dividing K")
    qcode = _code(qparam_dtype, "fq_int4_sym_tiled_group (qparams)")
    dev = ws[0].device
    n_total = sum(w.shape[0] for w in ws)
    tf = torch.empty(n_total * K, dtype=torch.bfloat16, device=dev) if forward else None
    tb = torch.empty(n_total * K, dtype=torch.bfloat16, device=dev) if backward else None
    scales = []
    lib = _lib.load()
    e = float(torch.finfo(torch.float32).eps) if eps is None else float(eps)
    n_off = 0
    with torch.cuda.device(dev):
        for w in ws:
            wc = w.contiguous()
            N = wc.shape[0]
            scale = torch.empty(N, K // group_size, dtype=torch.float32, device=dev)
            events = _fq_timer(f"per_group_tiled{int(forward) + int(backward)}", N, K, group_size, 2) if _fq_timer is not None else None
            if events:
                events[0].record()
            f_off = (128 if n_off else 0) if paired else n_off  # paired: the second member starts 128 columns in
            rc = lib.ttamd_fq_per_group_int4_sym_tiled_at_bf16(wc.data_ptr(), N, K, group_size, qcode, e,
                                                               tf.data_ptr() + 2 * K * f_off if forward else None, 1 if paired else 0,
                                                               _ptr(tb), n_total, n_off, scale.data_ptr(), _stream(w))
            if events:
                events[1].record()
            _lib.check(rc, "fq_int4_sym_tiled_group")
            scales.append(scale)
            n_off += N
    return tf, tb, scales


def tiled_linear_group_fwd(x: torch.Tensor, tiled: torch.Tensor, n_outs: Sequence[int],
                           biases: Optional[Sequence[Optional[torch.Tensor]]] = None, swiglu: bool = False):
    """-> [y_i [M, n_out_i]] = x @ Wd_i.T (+ bias_i) for weights stacked in the tiled layout, one launch.  ``swiglu`` (two
    members of equal width whose forward tiles are in the paired layout): ``silu(y_0) * y_1`` is appended, written by the
    same launch."""
    x = _bf16_2d(x, "tiled_linear_group_fwd")
    M, K = x.shape
    n = len(n_outs)
    if not 1 <= n <= _lib.GROUP_MAX or any(o <= 0 or o % 256 for o in n_outs):
        raise ValueError(f"tiled_linear_group_fwd: 1 to {_lib.GROUP_MAX} members with widths that are multiples of 256 (got {list(n_outs)})")
    if tiled.dtype != torch.bfloat16 or tiled.numel() != sum(n_outs) * K or not tiled.is_contiguous():
        raise ValueError(f"tiled_linear_group_fwd: the tiled weights must be a contiguous bfloat16 tensor of {sum(n_outs)} x {K} elements")
    if swiglu and (n != 2 or n_outs[0] != n_outs[1]):
        raise ValueError("tiled_linear_group_fwd: swiglu takes the gate and the up projection, two members of equal width")
    ys = [torch.empty(M, o, dtype=torch.bfloat16, device=x.device) for o in n_outs]
    act = torch.empty(M, n_outs[0], dtype=torch.bfloat16, device=x.device) if swiglu else None
    bs = [None] * n if biases is None else [None if b is None else b.contiguous() for b in biases]
    for b, o in zip(bs, n_outs):
        if b is not None and (b.dtype != torch.bfloat16 or b.numel() != o):
            raise ValueError(f"tiled_linear_group_fwd: a bias must be bfloat16 with {o} elements")
    c_n = (ctypes.c_int64 * n)(*n_outs)
    c_b = (ctypes.c_void_p * n)(*[_ptr(b) for b in bs])
    c_y = (ctypes.c_void_p * n)(*[y.data_ptr() for y in ys])
    lib = _lib.load()
    with torch.cuda.device(x.device):
        events = _gemm_timer("tiled", M, sum(n_outs), K, 0) if _gemm_timer is not None else None
        if events:
            events[0].record()
        rc = lib.ttamd_tiled_linear_group_fwd_bf16(x.data_ptr(), tiled.data_ptr(), n, c_n, c_b, c_y, _ptr(act), M, K, _stream(x))
        if events:
            events[1].record()
    _lib.check(rc, "tiled_linear_group_fwd")
    return ys + [act] if swiglu else ys


def tiled_linear_group_dx(gys: Sequence[torch.Tensor], tiled_t: torch.Tensor, K: int) -> torch.Tensor:
    """-> gx [M, K] = sum_i gy_i @ Wd_i for the transposed tiles of the stacked weights, one launch."""
    gys = [_bf16_2d(g, "tiled_linear_group_dx") for g in gys]
    M = gys[0].shape[0]
    n = len(gys)
    n_outs = [g.shape[1] for g in gys]
    if not 1 <= n <= _lib.GROUP_MAX or any(g.shape[0] != M for g in gys) or any(o % 64 for o in n_outs) or K % 64:
        raise ValueError(f"tiled_linear_group_dx: 1 to {_lib.GROUP_MAX} gradients over the same rows, widths and K multiples of 64")
    if tiled_t.dtype != torch.bfloat16 or tiled_t.numel() != sum(n_outs) * K or not tiled_t.is_contiguous():
        raise ValueError(f"tiled_linear_group_dx: the tiled weights must be a contiguous bfloat16 tensor of {sum(n_outs)} x {K} elements")
    gx = torch.empty(M, K, dtype=torch.bfloat16, device=gys[0].device)
    c_n = (ctypes.c_int64 * n)(*n_outs)
    c_g = (ctypes.c_void_p * n)(*[g.data_ptr() for g in gys])
    lib = _lib.load()
    with torch.cuda.device(gx.device):
        events = _gemm_timer("tiled", M, K, sum(n_outs), 0) if _gemm_timer is not None else None
        if events:
            events[0].record()
        rc = lib.ttamd_tiled_linear_group_dx_bf16(c_g, c_n, n, tiled_t.data_ptr(), gx.data_ptr(), M, K, _stream(gx))
        if events:
            events[1].record()
    _lib.check(rc, "tiled_linear_group_dx")
    return gx


def tiled_linear(x: torch.Tensor, tiled: torch.Tensor, n_out: int, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y [M, n_out] = x [M, k] @ Wd.T (+ bias) for a bf16 weight ``Wd`` [n_out, k] held in the tiled layout."""
    x = _bf16_2d(x, "tiled_linear")
    M, K = x.shape
    if tiled.dtype != torch.bfloat16 or tiled.numel() != n_out * K or not tiled.is_contiguous():
        raise ValueError(f"tiled_linear: the tiled weight must be a contiguous bfloat16 tensor of {n_out} x {K} elements")
    if bias is not None:
        bias = bias.contiguous()
        if bias.dtype != torch.bfloat16 or bias.numel() != n_out:
            raise ValueError(f"tiled_linear: bias must be bfloat16 with {n_out} elements")
    y = torch.empty(M, n_out, dtype=torch.bfloat16, device=x.device)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        events = _gemm_timer("tiled", M, n_out, K, 0) if _gemm_timer is not None else None
        if events:
            events[0].record()
        rc = lib.ttamd_tiled_linear_bf16(x.data_ptr(), tiled.data_ptr(), _ptr(bias), y.data_ptr(), M, n_out, K, _stream(x))
        if events:
            events[1].record()
    _lib.check(rc, "tiled_linear")
    return y


def tiled_lora_linear(x: torch.Tensor, tiled: torch.Tensor, n_out: int, lx: torch.Tensor, lw: torch.Tensor, lscale: float,
                      lw_row_major: bool, bias: Optional[torch.Tensor] = None, nf4_forward: bool = False) -> torch.Tensor:
    """``tiled_linear`` with a low-rank adapter in the GEMM's epilogue: ``y = x @ Wd.T (+ bias) + lscale * lx @ lw.T``
    with ``lw`` [n_out, r] (``lw_row_major``, the forward: ``lora_b``) or ``lw.T`` given as [r, n_out] (the grad-input:
    ``lora_a``).  ``tiled`` may be longer than n_out * K elements (a workspace whose head holds the tiles);
    ``nf4_forward``: the tiles are an NF4 weight's expansion kept from an earlier call (what a GEMM timer is told)."""
    x = _bf16_2d(x, "tiled_lora_linear")
    lx = _bf16_2d(lx, "tiled_lora_linear")
    lw = _bf16_2d(lw, "tiled_lora_linear")
    M, K = x.shape
    r = lx.shape[1]
    if tiled.numel() * tiled.element_size() < 2 * n_out * K or not tiled.is_contiguous():
        raise ValueError(f"tiled_lora_linear: the tiled weight must be contiguous and hold {n_out} x {K} bfloat16 elements")
    if lx.shape[0] != M or tuple(lw.shape) != ((n_out, r) if lw_row_major else (r, n_out)) or r % 8 != 0 or not 0 < r <= 64:
        raise ValueError(f"tiled_lora_linear: adapter operands {tuple(lx.shape)} / {tuple(lw.shape)} do not fit M={M}, n_out={n_out} "
                         "(rank: a multiple of 8, at most 64)")
    if bias is not None:
        bias = bias.contiguous()
        if bias.dtype != torch.bfloat16 or bias.numel() != n_out:
            raise ValueError(f"tiled_lora_linear: bias must be bfloat16 with {n_out} elements")
    y = torch.empty(M, n_out, dtype=torch.bfloat16, device=x.device)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        events = None
        if _gemm_timer is not None:
            events = _gemm_timer("fwd", M, n_out, K, r) if nf4_forward else _gemm_timer("tiled", M, n_out, K, 0)
        if events:
            events[0].record()
        rc = lib.ttamd_tiled_lora_linear_bf16(x.data_ptr(), tiled.data_ptr(), lx.data_ptr(), lw.data_ptr(), 1 if lw_row_major else 0, r,
                                              float(lscale), _ptr(bias), y.data_ptr(), M, n_out, K, _stream(x))
        if events:
            events[1].record()
    _lib.check(rc, "tiled_lora_linear")
    return y


def tiled_linear_dx(gy: torch.Tensor, tiled_fwd: torch.Tensor, K: int, gh: Optional[torch.Tensor] = None,
                    lora_a: Optional[torch.Tensor] = None, nf4_backward: bool = False) -> torch.Tensor:
    """``gx = gy @ Wd (+ gh @ lora_a)`` with ``Wd`` [N, K] given as the FORWARD tiles (what ``tiled_linear`` / the expanded
    NF4 forward read): the grad-input without a transposed copy of the weight, bit-equal to the launch on tiles of
    ``Wd.T``.  ``tiled_fwd`` may be longer than N * K elements (a workspace whose head holds the tiles)."""
    gy = _bf16_2d(gy, "tiled_linear_dx")
    M, N = gy.shape
    if tiled_fwd.numel() * tiled_fwd.element_size() < 2 * N * K or not tiled_fwd.is_contiguous():
        raise ValueError(f"tiled_linear_dx: the tiled weight must be contiguous and hold {N} x {K} bfloat16 elements")
    r = 0
    if gh is not None:
        gh = _bf16_2d(gh, "tiled_linear_dx")
        lora_a = _bf16_2d(lora_a, "tiled_linear_dx")
        r = gh.shape[1]
        if gh.shape[0] != M or tuple(lora_a.shape) != (r, K) or r % 8 != 0 or not 0 < r <= 64:
            raise ValueError(f"tiled_linear_dx: adapter operands {tuple(gh.shape)} / {tuple(lora_a.shape)} do not fit M={M}, K={K}")
    gx = torch.empty(M, K, dtype=torch.bfloat16, device=gy.device)
    lib = _lib.load()
    with _on_device(gy.device):
        # an installed timer books the call as what it is: the grad-input of an NF4 layer, or a GEMM on fake-quantised tiles
        events = None
        if _gemm_timer is not None:
            events = _gemm_timer("bwd", M, N, K, r, on_tiles=True) if nf4_backward else _gemm_timer("tiled", M, K, N, 0)
        if events:
            events[0].record()
        rc = lib.ttamd_tiled_linear_dx_bf16(gy.data_ptr(), tiled_fwd.data_ptr(), _ptr(gh), _ptr(lora_a), r, gx.data_ptr(), M, N, K,
                                            _stream(gy))
        if events:
            events[1].record()
    _lib.check(rc, "tiled_linear_dx")
    return gx


def gemm_tn_applies(M: int, N: int, K: int) -> bool:
    """Shapes ``gemm_tn`` serves: M a multiple of 32, N and K multiples of 256."""
    return bool(_lib.load().ttamd_gemm_tn_applies(M, N, K))


# The tiles of a weight-gradient launch beyond its last whole round of 256 get their contraction cut into slices when the
# library is given room for the partial tiles (False: never, the launch of the plain entry points).
TN_TAIL_SLICES = True


def _tn_workspace(lib, M: int, n_total: int, K: int, device):
    nbytes = int(lib.ttamd_gemm_tn_workspace_bytes(M, n_total, K)) if TN_TAIL_SLICES else 0
    if nbytes == 0:
        return None, 0
    return torch.empty(nbytes // 4, dtype=torch.float32, device=device), nbytes


def gemm_tn(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """a [M, N], b [M, K] bf16 -> a.T @ b [N, K] bf16 (fp32 accumulation): the weight gradient of a linear layer."""
    a = _bf16_2d(a, "gemm_tn")
    b = _bf16_2d(b, "gemm_tn")
    M, N = a.shape
    if b.shape[0] != M:
        raise ValueError(f"gemm_tn: a has {M} rows, b {b.shape[0]}")
    K = b.shape[1]
    c = torch.empty(N, K, dtype=torch.bfloat16, device=a.device)
    lib = _lib.load()
    ws, ws_bytes = _tn_workspace(lib, M, N, K, a.device)
    with torch.cuda.device(a.device):
        events = _gemm_timer("tn", M, N, K, 0) if _gemm_timer is not None else None
        if events:
            events[0].record()
        rc = lib.ttamd_gemm_tn_ws_bf16(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, _ptr(ws), ws_bytes, _stream(a))
        if events:
            events[1].record()
    _lib.check(rc, "gemm_tn")
    return c


def gemm_tn_group(a_list: Sequence[torch.Tensor], b: torch.Tensor) -> List[torch.Tensor]:
    """``[a.T @ b for a in a_list]`` (each ``a`` [M, N_i], ``b`` [M, K], bf16) as one launch: the weight gradients of layers
    with a common input.  Each result carries the bits ``gemm_tn(a, b)`` gives wherever neither launch cuts the tile's
    contraction into slices (``TN_TAIL_SLICES``: the tiles of a launch's last partial round)."""
    b = _bf16_2d(b, "gemm_tn_group")
    a_list = [_bf16_2d(a, "gemm_tn_group") for a in a_list]
    M, K = b.shape
    n = len(a_list)
    if not 1 <= n <= _lib.GROUP_MAX:
        raise ValueError(f"gemm_tn_group: {n} members (1 .. {_lib.GROUP_MAX})")
    for a in a_list:
        if a.shape[0] != M or a.device != b.device:
            raise ValueError(f"gemm_tn_group: a {tuple(a.shape)} on {a.device} does not go with b {tuple(b.shape)} on {b.device}")
    cs = [torch.empty(a.shape[1], K, dtype=torch.bfloat16, device=b.device) for a in a_list]
    a_ptrs = (ctypes.c_void_p * n)(*[a.data_ptr() for a in a_list])
    c_ptrs = (ctypes.c_void_p * n)(*[c.data_ptr() for c in cs])
    widths = (ctypes.c_int64 * n)(*[a.shape[1] for a in a_list])
    lib = _lib.load()
    ws, ws_bytes = _tn_workspace(lib, M, sum(a.shape[1] for a in a_list), K, b.device)
    with torch.cuda.device(b.device):
        events = _gemm_timer("tn", M, sum(a.shape[1] for a in a_list), K, 0) if _gemm_timer is not None else None
        if events:
            events[0].record()
        rc = lib.ttamd_gemm_tn_group_ws_bf16(a_ptrs, b.data_ptr(), c_ptrs, n, M, widths, K, _ptr(ws), ws_bytes, _stream(b))
        if events:
            events[1].record()
    _lib.check(rc, "gemm_tn_group")
    return cs


def quantize_per_group_int4(w: torch.Tensor, group_size: int, qparam_dtype: torch.dtype = torch.float32,
                            eps: Optional[float] = None):
    """w [rows, K] -> (int8 tensor of int4 values, scale fp32 [rows, K/g], zeros fp32 [rows, K/g])"""
    _need_gpu(w, "quantize_per_group_int4")
    code = _code(w.dtype, "quantize_per_group_int4")
    qcode = _code(qparam_dtype, "quantize_per_group_int4 (qparams)")
    wc = w.contiguous()
    K = wc.shape[-1]
    rows = wc.numel() // K
    q = torch.empty(wc.shape, dtype=torch.int8, device=w.device)
    scale = torch.empty(rows, K // max(group_size, 1), dtype=torch.float32, device=w.device)
    zeros = torch.empty_like(scale)
    lib = _lib.load()
    with torch.cuda.device(w.device):
        rc = lib.ttamd_quantize_per_group_int4_conv(wc.data_ptr(), code, rows, K, group_size, qcode, q.data_ptr(), scale.data_ptr(),
                                                    zeros.data_ptr(), _conventions(eps_per_group_sym=eps), _stream(w))
    _lib.check(rc, "quantize_per_group_int4")
    return q, scale, zeros


def fq_per_group_uint4_asym(w: torch.Tensor, group_size: int, qparam_dtype: torch.dtype = torch.bfloat16,
                            want_qparams: bool = True, min_scale: Optional[float] = None, clamp_range_first: bool = False):
    """Weight-only int4 scheme (asymmetric uint4, floating-point zero point):
    w [..., K] -> (fake-quantised w, scale fp32 [rows, K/g] | None, zero_point fp32 [rows, K/g] | None);
    the qparams hold values already rounded to ``qparam_dtype``.  ``min_scale`` (None = 1e-6) bounds the scale from below;
    ``clamp_range_first`` applies that bound to ``max - min`` before the division by 15 instead of to the quotient."""
    _need_gpu(w, "fq_per_group_uint4_asym")
    code = _code(w.dtype, "fq_per_group_uint4_asym")
    qcode = _code(qparam_dtype, "fq_per_group_uint4_asym (qparams)")
    wc = w.contiguous()
    K = wc.shape[-1]
    rows = wc.numel() // K
    out = torch.empty_like(wc)
    scale = torch.empty(rows, K // max(group_size, 1), dtype=torch.float32, device=w.device) if want_qparams else None
    zero = torch.empty_like(scale) if want_qparams else None
    lib = _lib.load()
    with torch.cuda.device(w.device):
        events = _fq_timer("per_group", rows, K, group_size, wc.element_size()) if _fq_timer is not None else None
        if events:
            events[0].record()
        rc = lib.ttamd_fq_per_group_uint4_asym_conv(
            wc.data_ptr(), code, rows, K, group_size, qcode, out.data_ptr(), _ptr(scale), _ptr(zero),
            _conventions(min_scale_uint4=min_scale, clamp_range_first=clamp_range_first), _stream(w))
        if events:
            events[1].record()
    _lib.check(rc, "fq_per_group_uint4_asym")
    return out, scale, zero


def quantize_per_group_uint4(w: torch.Tensor, group_size: int, qparam_dtype: torch.dtype = torch.bfloat16,
                             min_scale: Optional[float] = None, clamp_range_first: bool = False):
    """w [rows, K] -> (uint8 [rows, K/2], two codes per byte with the even element in the high nibble,
    scale fp32 [rows, K/g], zero_point fp32 [rows, K/g])"""
    _need_gpu(w, "quantize_per_group_uint4")
    code = _code(w.dtype, "quantize_per_group_uint4")
    qcode = _code(qparam_dtype, "quantize_per_group_uint4 (qparams)")
    if w.dim() != 2:
        raise ValueError(f"quantize_per_group_uint4: expected a 2-D weight, got {tuple(w.shape)}")
    wc = w.contiguous()
    rows, K = wc.shape
    q = torch.empty(rows, K // 2, dtype=torch.uint8, device=w.device)
    scale = torch.empty(rows, K // max(group_size, 1), dtype=torch.float32, device=w.device)
    zero = torch.empty_like(scale)
    lib = _lib.load()
    with torch.cuda.device(w.device):
        rc = lib.ttamd_quantize_per_group_uint4_conv(
            wc.data_ptr(), code, rows, K, group_size, qcode, q.data_ptr(), scale.data_ptr(), zero.data_ptr(),
            _conventions(min_scale_uint4=min_scale, clamp_range_first=clamp_range_first), _stream(w))
    _lib.check(rc, "quantize_per_group_uint4")
    return q, scale, zero


def dequantize_per_group_uint4(q: torch.Tensor, scale: torch.Tensor, zero: torch.Tensor, group_size: int,
                               dtype: torch.dtype) -> torch.Tensor:
    """q [rows, K/2] uint8 (packed codes), scale / zero fp32 [rows, K/g] -> dtype((q - 8) * scale + zero) [rows, K]"""
    _need_gpu(q, "dequantize_per_group_uint4")
    code = _code(dtype, "dequantize_per_group_uint4")
    if q.dtype != torch.uint8 or q.dim() != 2:
        raise TypeError(f"dequantize_per_group_uint4: q must be a 2-D uint8 tensor, got {tuple(q.shape)} {q.dtype}")
    qc = q.contiguous()
    rows, K = qc.shape[0], qc.shape[1] * 2
    sc = scale.to(torch.float32).contiguous()
    zc = zero.to(torch.float32).contiguous()
    if sc.numel() != rows * (K // max(group_size, 1)) or zc.numel() != sc.numel():
        raise ValueError("dequantize_per_group_uint4: scale / zero must have rows * K / group_size elements")
    out = torch.empty(rows, K, dtype=dtype, device=q.device)
    lib = _lib.load()
    with torch.cuda.device(q.device):
        rc = lib.ttamd_dequantize_per_group_uint4(qc.data_ptr(), sc.data_ptr(), zc.data_ptr(), code, rows, K, group_size,
                                                  out.data_ptr(), _stream(q))
    _lib.check(rc, "dequantize_per_group_uint4")
    return out


def dequantize_per_group_int4(q: torch.Tensor, scale: torch.Tensor, zeros: Optional[torch.Tensor], group_size: int,
                              dtype: torch.dtype) -> torch.Tensor:
    """q [rows, K] int8 (int4 values), scale/zeros fp32 [rows, K/g] -> dtype((q - zeros) * scale) [rows, K]"""
    _need_gpu(q, "dequantize_per_group_int4")
    code = _code(dtype, "dequantize_per_group_int4")
    if q.dtype != torch.int8 or q.dim() != 2:
        raise TypeError(f"dequantize_per_group_int4: q must be a 2-D int8 tensor, got {tuple(q.shape)} {q.dtype}")
    qc = q.contiguous()
    rows, K = qc.shape
    sc = scale.to(torch.float32).contiguous()
    zc = zeros.to(torch.float32).contiguous() if zeros is not None else None
    if sc.numel() != rows * (K // max(group_size, 1)) or (zc is not None and zc.numel() != sc.numel()):
        raise ValueError("dequantize_per_group_int4: scale / zeros must have rows * K / group_size elements")
    out = torch.empty(rows, K, dtype=dtype, device=q.device)
    lib = _lib.load()
    with torch.cuda.device(q.device):
        rc = lib.ttamd_dequantize_per_group_int4(qc.data_ptr(), sc.data_ptr(), _ptr(zc), code, rows, K, group_size, out.data_ptr(),
                                                 _stream(q))
    _lib.check(rc, "dequantize_per_group_int4")
    return out


# ---------------------------------------------------------------------------------------------------
# neighbours of the quantized linears in a decoder layer: RMSNorm, rotary embedding, SwiGLU gate
# ---------------------------------------------------------------------------------------------------
def _bf16_any(t: torch.Tensor, what: str) -> torch.Tensor:
    _need_gpu(t, what)
    if t.dtype != torch.bfloat16:
        raise TypeError(f"{what}: expected a bfloat16 tensor, got {t.dtype}")
    return t.contiguous()


def rms_norm_fwd(x: torch.Tensor, scale: torch.Tensor, eps: float):
    """x [..., D] bf16, scale [D] bf16 -> (y like x, rstd fp32 [rows])"""
    xc = _bf16_any(x, "rms_norm_fwd: x")
    sc = _bf16_any(scale, "rms_norm_fwd: scale")
    D = xc.shape[-1]
    rows = xc.numel() // D
    y = torch.empty_like(xc)
    rstd = torch.empty(rows, dtype=torch.float32, device=x.device)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        rc = lib.ttamd_rms_norm_fwd_bf16(xc.data_ptr(), sc.data_ptr(), float(eps), y.data_ptr(), rstd.data_ptr(), rows, D, _stream(x))
    _lib.check(rc, "rms_norm_fwd")
    return y, rstd


def add_rms_norm_fwd(x: torch.Tensor, residual: torch.Tensor, scale: torch.Tensor, eps: float):
    """-> (h = x + residual, y = RMSNorm(h), rstd): the addition of the residual stream and the norm that follows it in
    one pass; the bits of ``x + residual`` followed by ``rms_norm_fwd``."""
    xc = _bf16_any(x, "add_rms_norm_fwd: x")
    rc_ = _bf16_any(residual, "add_rms_norm_fwd: residual")
    sc = _bf16_any(scale, "add_rms_norm_fwd: scale")
    if xc.shape != rc_.shape:
        raise ValueError(f"add_rms_norm_fwd: x {tuple(xc.shape)} and residual {tuple(rc_.shape)} differ in shape")
    D = xc.shape[-1]
    rows = xc.numel() // D
    h = torch.empty_like(xc)
    y = torch.empty_like(xc)
    rstd = torch.empty(rows, dtype=torch.float32, device=x.device)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        rc = lib.ttamd_add_rms_norm_fwd_bf16(xc.data_ptr(), rc_.data_ptr(), sc.data_ptr(), float(eps), h.data_ptr(), y.data_ptr(),
                                             rstd.data_ptr(), rows, D, _stream(x))
    _lib.check(rc, "add_rms_norm_fwd")
    return h, y, rstd


def rms_norm_bwd(gy: torch.Tensor, x: torch.Tensor, scale: torch.Tensor, rstd: torch.Tensor, want_gscale: bool,
                 g_add: Optional[torch.Tensor] = None):
    """-> (gx like x, gscale [D] bf16 | None); ``g_add`` (like x): a gradient that reaches x on another way, added to gx in
    the same pass (``bf16(bf16(gx) + g_add)``)."""
    gc = _bf16_any(gy, "rms_norm_bwd: gy")
    xc = _bf16_any(x, "rms_norm_bwd: x")
    sc = _bf16_any(scale, "rms_norm_bwd: scale")
    D = xc.shape[-1]
    rows = xc.numel() // D
    gx = torch.empty_like(xc)
    lib = _lib.load()
    gscale = torch.empty(D, dtype=torch.bfloat16, device=x.device) if want_gscale else None
    nbytes = lib.ttamd_rms_norm_bwd_workspace_bytes(D) if want_gscale else 0
    ws = _workspace(nbytes, x.device) if want_gscale else None
    ga = None
    if g_add is not None:
        ga = _bf16_any(g_add, "rms_norm_bwd: g_add")
        if ga.shape != xc.shape:
            raise ValueError(f"rms_norm_bwd: g_add {tuple(ga.shape)} and x {tuple(xc.shape)} differ in shape")
    with torch.cuda.device(x.device):
        rc = lib.ttamd_rms_norm_bwd_add_bf16(gc.data_ptr(), xc.data_ptr(), sc.data_ptr(), rstd.data_ptr(), _ptr(ga), gx.data_ptr(),
                                             _ptr(gscale), rows, D, _ptr(ws), nbytes, _stream(x))
    _lib.check(rc, "rms_norm_bwd")
    return gx, gscale


def rope(x: torch.Tensor, cache: torch.Tensor, inverse: bool = False) -> torch.Tensor:
    """x [b, s, n_h, h_d] bf16, cache [s, h_d/2, 2] fp32 -> rotated x (inverse: by the negative angle)"""
    xc = _bf16_any(x, "rope: x")
    if xc.dim() != 4:
        raise ValueError(f"rope: expected [b, s, n_h, h_d], got {tuple(x.shape)}")
    b, s, nh, hd = xc.shape
    _need_gpu(cache, "rope: cache")
    if cache.dtype != torch.float32 or cache.numel() < s * hd or cache.shape[-1] != 2 or cache.shape[-2] != hd // 2:
        raise ValueError(f"rope: cache must be fp32 [>= {s}, {hd // 2}, 2], got {tuple(cache.shape)} {cache.dtype}")
    cc = cache.contiguous()
    y = torch.empty_like(xc)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        rc = lib.ttamd_rope_bf16(xc.data_ptr(), cc.data_ptr(), y.data_ptr(), b, s, nh, hd, int(bool(inverse)), _stream(x))
    _lib.check(rc, "rope")
    return y


def repeat_kv(x: torch.Tensor, rep: int) -> torch.Tensor:
    """x [b, s, n_kv, h_d] bf16 -> [b, s, n_kv * rep, h_d]: every key / value head ``rep`` times in a row."""
    xc = _bf16_any(x, "repeat_kv: x")
    if xc.dim() != 4 or rep < 1:
        raise ValueError(f"repeat_kv: expected [b, s, n_kv, h_d] and rep >= 1, got {tuple(x.shape)}, rep={rep}")
    b, s, nkv, hd = xc.shape
    y = torch.empty(b, s, nkv * rep, hd, dtype=torch.bfloat16, device=xc.device)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        rc = lib.ttamd_repeat_kv_bf16(xc.data_ptr(), y.data_ptr(), b * s, nkv, rep, hd, _stream(x))
    _lib.check(rc, "repeat_kv")
    return y


def repeat_kv_bwd(gy: torch.Tensor, rep: int) -> torch.Tensor:
    """gy [b, s, n_kv * rep, h_d] bf16 -> [b, s, n_kv, h_d]: the sum over each head's ``rep`` copies."""
    g = _bf16_any(gy, "repeat_kv_bwd: gy")
    if g.dim() != 4 or rep < 1 or g.shape[2] % rep:
        raise ValueError(f"repeat_kv_bwd: expected [b, s, n_kv * rep, h_d], got {tuple(gy.shape)}, rep={rep}")
    b, s, nh, hd = g.shape
    gx = torch.empty(b, s, nh // rep, hd, dtype=torch.bfloat16, device=g.device)
    lib = _lib.load()
    with torch.cuda.device(gy.device):
        rc = lib.ttamd_repeat_kv_bwd_bf16(g.data_ptr(), gx.data_ptr(), b * s, nh // rep, rep, hd, _stream(gy))
    _lib.check(rc, "repeat_kv_bwd")
    return gx


def _rope_cache_arg(cache: torch.Tensor, s: int, hd: int, who: str) -> torch.Tensor:
    _need_gpu(cache, f"{who}: cache")
    if cache.dtype != torch.float32 or cache.numel() < s * hd or cache.shape[-1] != 2 or cache.shape[-2] != hd // 2:
        raise ValueError(f"{who}: cache must be fp32 [>= {s}, {hd // 2}, 2], got {tuple(cache.shape)} {cache.dtype}")
    return cache.contiguous()


def _qkv_shapes(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, n_kv: Optional[int], who: str):
    if q.dim() != 4 or k.dim() != 4 or v.shape != k.shape or q.shape[:2] != k.shape[:2] or q.shape[3] != k.shape[3]:
        raise ValueError(f"{who}: expected [b, s, n_h, h_d] and two [b, s, n_kv, h_d], got {tuple(q.shape)}, {tuple(k.shape)}, {tuple(v.shape)}")
    b, s, nh, hd = q.shape
    nkv = k.shape[2] if n_kv is None else n_kv
    if nkv < 1 or nh % nkv or (n_kv is not None and k.shape[2] != nh):
        raise ValueError(f"{who}: {nh} query heads against {nkv} key / value heads (tensors {tuple(q.shape)}, {tuple(k.shape)})")
    return b, s, nh, nkv, hd


def qkv_rope_repeat(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cache: torch.Tensor):
    """``rope(q)``, ``repeat_kv(rope(k), n_h // n_kv)``, ``repeat_kv(v, n_h // n_kv)`` from one launch; q ``[b, s, n_h, h_d]``,
    k and v ``[b, s, n_kv, h_d]`` bf16, cache ``[s, h_d/2, 2]`` fp32.  The bits of :func:`rope` and :func:`repeat_kv`."""
    qc, kc, vc = _bf16_any(q, "qkv_rope_repeat: q"), _bf16_any(k, "qkv_rope_repeat: k"), _bf16_any(v, "qkv_rope_repeat: v")
    b, s, nh, nkv, hd = _qkv_shapes(qc, kc, vc, None, "qkv_rope_repeat")
    cc = _rope_cache_arg(cache, s, hd, "qkv_rope_repeat")
    qo, ko, vo = torch.empty_like(qc), torch.empty_like(qc), torch.empty_like(qc)
    lib = _lib.load()
    with torch.cuda.device(q.device):
        rc = lib.ttamd_qkv_rope_repeat_bf16(qc.data_ptr(), kc.data_ptr(), vc.data_ptr(), cc.data_ptr(), qo.data_ptr(),
                                            ko.data_ptr(), vo.data_ptr(), b, s, nh, nkv, hd, _stream(q))
    _lib.check(rc, "qkv_rope_repeat")
    return qo, ko, vo


def qkv_rope_repeat_bwd(gq_out: torch.Tensor, gk_out: torch.Tensor, gv_out: torch.Tensor, cache: torch.Tensor, n_kv: int):
    """The gradients of q, k, v of :func:`qkv_rope_repeat` from those of its three outputs (each ``[b, s, n_h, h_d]``)."""
    a, bb, c = (_bf16_any(gq_out, "qkv_rope_repeat_bwd: gq"), _bf16_any(gk_out, "qkv_rope_repeat_bwd: gk"),
                _bf16_any(gv_out, "qkv_rope_repeat_bwd: gv"))
    b, s, nh, nkv, hd = _qkv_shapes(a, bb, c, n_kv, "qkv_rope_repeat_bwd")
    cc = _rope_cache_arg(cache, s, hd, "qkv_rope_repeat_bwd")
    gq = torch.empty_like(a)
    gk = torch.empty(b, s, nkv, hd, dtype=torch.bfloat16, device=a.device)
    gv = torch.empty_like(gk)
    lib = _lib.load()
    with torch.cuda.device(a.device):
        rc = lib.ttamd_qkv_rope_repeat_bwd_bf16(a.data_ptr(), bb.data_ptr(), c.data_ptr(), cc.data_ptr(), gq.data_ptr(),
                                                gk.data_ptr(), gv.data_ptr(), b, s, nh, nkv, hd, _stream(a))
    _lib.check(rc, "qkv_rope_repeat_bwd")
    return gq, gk, gv


def swiglu_fwd(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    g = _bf16_any(gate, "swiglu_fwd: gate")
    u = _bf16_any(up, "swiglu_fwd: up")
    if g.shape != u.shape:
        raise ValueError(f"swiglu_fwd: shapes differ: {tuple(g.shape)} vs {tuple(u.shape)}")
    out = torch.empty_like(g)
    lib = _lib.load()
    with torch.cuda.device(g.device):
        rc = lib.ttamd_swiglu_fwd_bf16(g.data_ptr(), u.data_ptr(), out.data_ptr(), g.numel(), _stream(g))
    _lib.check(rc, "swiglu_fwd")
    return out


def swiglu_bwd(gout: torch.Tensor, gate: torch.Tensor, up: torch.Tensor):
    go = _bf16_any(gout, "swiglu_bwd: gout")
    g = _bf16_any(gate, "swiglu_bwd: gate")
    u = _bf16_any(up, "swiglu_bwd: up")
    gg = torch.empty_like(g)
    gu = torch.empty_like(u)
    lib = _lib.load()
    with torch.cuda.device(g.device):
        rc = lib.ttamd_swiglu_bwd_bf16(go.data_ptr(), g.data_ptr(), u.data_ptr(), gg.data_ptr(), gu.data_ptr(), g.numel(), _stream(g))
    _lib.check(rc, "swiglu_bwd")
    return gg, gu


# ---------------------------------------------------------------------------------------------------
# DoRA over an NF4 base weight
# ---------------------------------------------------------------------------------------------------
def nf4_dora_weight_norm(qdata: torch.Tensor, block_scalers: torch.Tensor, N: int, K: int, lora_a: torch.Tensor,
                         lora_b: torch.Tensor, scale: float, magnitude: Optional[torch.Tensor] = None):
    """-> (weight_norm [N] bf16, magnitude / weight_norm [N] bf16 | None): row norms of D(W) + scale * B @ A"""
    _need_gpu(qdata, "nf4_dora_weight_norm")
    a = _bf16_2d(lora_a, "nf4_dora_weight_norm: lora_a")
    b = _bf16_2d(lora_b, "nf4_dora_weight_norm: lora_b")
    rank = a.shape[0]
    if a.shape != (rank, K) or b.shape != (N, rank):
        raise ValueError(f"nf4_dora_weight_norm: lora_a {tuple(a.shape)} / lora_b {tuple(b.shape)} do not fit [{N}, {K}]")
    mag = _bf16_any(magnitude, "nf4_dora_weight_norm: magnitude") if magnitude is not None else None
    norm = torch.empty(N, dtype=torch.bfloat16, device=qdata.device)
    mns = torch.empty(N, dtype=torch.bfloat16, device=qdata.device) if mag is not None else None
    lib = _lib.load()
    nbytes = lib.ttamd_dora_weight_norm_workspace_bytes(N, K)
    ws = _workspace(nbytes, qdata.device)
    with torch.cuda.device(qdata.device):
        rc = lib.ttamd_nf4_dora_weight_norm_bf16(qdata.data_ptr(), block_scalers.data_ptr(), a.data_ptr(), b.data_ptr(), rank,
                                                 float(scale), _ptr(mag), norm.data_ptr(), _ptr(mns), N, K, ws.data_ptr(), nbytes,
                                                 _stream(qdata))
    _lib.check(rc, "nf4_dora_weight_norm")
    return norm, mns


def dora_bwd_prologue(gy: torch.Tensor, out: torch.Tensor, mag_norm_scale: torch.Tensor, magnitude: torch.Tensor):
    """gy, out [M, N] bf16 -> (gy * mag_norm_scale [M, N] bf16, grad of magnitude [N] bf16)"""
    g = _bf16_2d(gy, "dora_bwd_prologue: gy")
    o = _bf16_2d(out, "dora_bwd_prologue: out")
    mns = _bf16_any(mag_norm_scale, "dora_bwd_prologue: mag_norm_scale")
    mag = _bf16_any(magnitude, "dora_bwd_prologue: magnitude")
    M, N = g.shape
    gy0 = torch.empty_like(g)
    gmag = torch.empty(N, dtype=torch.bfloat16, device=g.device)
    lib = _lib.load()
    nbytes = lib.ttamd_dora_bwd_workspace_bytes(N)
    ws = _workspace(nbytes, g.device)
    with torch.cuda.device(g.device):
        rc = lib.ttamd_dora_bwd_prologue_bf16(g.data_ptr(), o.data_ptr(), mns.data_ptr(), mag.data_ptr(), gy0.data_ptr(),
                                              gmag.data_ptr(), M, N, ws.data_ptr(), nbytes, _stream(g))
    _lib.check(rc, "dora_bwd_prologue")
    return gy0, gmag


def cross_entropy_fwd_bwd(logits: torch.Tensor, target: torch.Tensor, ignore_index: int = -100, grad_scale: float = 1.0):
    """logits [rows, V] bf16, target [rows] int64 -> (per-row loss fp32 [rows], grad_scale * dloss/dlogits bf16 [rows, V])"""
    lg = _bf16_2d(logits, "cross_entropy_fwd_bwd: logits")
    _need_gpu(target, "cross_entropy_fwd_bwd: target")
    if target.dtype != torch.int64 or target.shape != (lg.shape[0],):
        raise TypeError(f"cross_entropy_fwd_bwd: target must be int64 [{lg.shape[0]}], got {tuple(target.shape)} {target.dtype}")
    tg = target.contiguous()
    rows, V = lg.shape
    loss = torch.empty(rows, dtype=torch.float32, device=lg.device)
    grad = torch.empty_like(lg)
    lib = _lib.load()
    with torch.cuda.device(lg.device):
        rc = lib.ttamd_cross_entropy_fwd_bwd_bf16(lg.data_ptr(), tg.data_ptr(), int(ignore_index), float(grad_scale), loss.data_ptr(),
                                                  grad.data_ptr(), rows, V, _stream(lg))
    _lib.check(rc, "cross_entropy_fwd_bwd")
    return loss, grad
