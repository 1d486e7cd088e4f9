"""State-dict hooks that strip NF4 from checkpoints: every ``NF4Tensor`` in ``module.state_dict()`` is replaced
by its dequantised dense tensor, optionally moved to the CPU.  Same contract as
``reparametrize_as_dtype_state_dict_post_hook`` / ``_register_reparametrize_state_dict_hooks`` in the reference
(``torchtune/modules/common_utils.py:24-59,206-237``); the dequantisation is the HIP kernel."""
from __future__ import annotations

import os
import sys
import tempfile
from functools import partial
from typing import Any, Dict

import torch
from torch import nn

from ..nf4_tensor import NF4Tensor

# The switch of the reference (``torchtune/modules/common_utils.py:21``): True makes
# ``_register_reparametrize_state_dict_hooks`` install the hook that keeps the dense checkpoint out of host RAM.
_use_low_cpu_ram: bool = False


# Offloaded weights land in pinned (page-locked) host memory, written by the dequantise kernel itself over PCIe.
# Set to False to get ordinary pageable tensors instead: the kernel then writes into one reusable pinned staging
# buffer and the host copies it out (for hosts that cannot lock a whole checkpoint).
PINNED_OFFLOAD = True

_staging: Dict[Any, torch.Tensor] = {}


def _staging_buffer(numel: int, dtype: torch.dtype) -> torch.Tensor:
    buf = _staging.get(dtype)
    if buf is None or buf.numel() < numel:
        buf = _staging[dtype] = torch.empty(numel, dtype=dtype, pin_memory=True)
    return buf[:numel]


def reparametrize_as_dtype_state_dict_post_hook(
    model: nn.Module,
    state_dict: Dict[str, Any],
    *args: Any,
    dtype: torch.dtype = torch.bfloat16,
    offload_to_cpu: bool = True,
    **kwargs: Any,
) -> None:
    """State-dict post hook: NF4 entries become dense ``dtype`` tensors (on the CPU if ``offload_to_cpu``).

    With ``offload_to_cpu`` no dense copy is made on the GPU: the dequantise kernel reads the packed weight from
    HBM and stores the dense values straight into host memory, so a checkpoint moves at PCIe speed."""
    wrote_to_host = None
    for k, v in state_dict.items():
        if not isinstance(v, NF4Tensor):
            continue
        if not (offload_to_cpu and v.quantized_data.is_cuda):
            dense = v.to(dtype)
            state_dict[k] = dense.cpu() if offload_to_cpu else dense
            continue
        wrote_to_host = v.quantized_data.device
        if PINNED_OFFLOAD:
            host = torch.empty(v.shape, dtype=dtype, pin_memory=True)
            if dtype == v.dtype:
                v.get_original_weight(out=host)
            else:
                host.copy_(v.get_original_weight().to(dtype), non_blocking=True)
        else:
            stage = _staging_buffer(v.numel(), v.dtype)
            v.get_original_weight(out=stage)
            torch.cuda.current_stream(wrote_to_host).synchronize()
            host = torch.empty(v.shape, dtype=dtype)
            host.view(-1).copy_(stage)
        state_dict[k] = host
    if wrote_to_host is not None:
        torch.cuda.current_stream(wrote_to_host).synchronize()


def _low_ram_reparametrize_as_dtype_state_dict_post_hook(
    model: nn.Module,
    state_dict: Dict[str, Any],
    *args: Any,
    dtype: torch.dtype = torch.bfloat16,
    offload_to_cpu: bool = True,
    **kwargs: Any,
) -> None:
    """The same replacement of NF4 entries for hosts whose RAM cannot hold the dense checkpoint
    (``torchtune/modules/common_utils.py:136-203``): every entry of the state dict ends up in ONE file-backed shared
    mapping, so the kernel of the operating system can write the pages back to disk instead of keeping them.

    The reference gets there through fake tensors, ``torch.save(skip_data)`` and ``torch.load(mmap=True)``; here the
    layout is computed directly: one temporary file of the total size is mapped (``MAP_SHARED``), each NF4 weight is
    dequantised by the HIP kernel into a reusable pinned staging buffer of one weight's size and copied into its slice
    of the mapping, every other entry is copied as it is.  The file is unlinked as soon as it is mapped, so nothing is
    left behind when the tensors are released.  Without ``offload_to_cpu`` there is nothing to keep out of host RAM and
    the ordinary hook runs."""
    if not offload_to_cpu:
        return reparametrize_as_dtype_state_dict_post_hook(model, state_dict, *args, dtype=dtype, offload_to_cpu=False, **kwargs)
    layout = []
    total = 0
    for k, v in state_dict.items():
        out_dtype = dtype if isinstance(v, NF4Tensor) else v.dtype
        nbytes = v.numel() * torch.empty((), dtype=out_dtype).element_size()
        layout.append((k, out_dtype, total, nbytes))
        total += (nbytes + 63) // 64 * 64
    if total == 0:
        return
    fd, path = tempfile.mkstemp(prefix="torchtune_amd_state_dict_", suffix=".bin")
    try:
        os.ftruncate(fd, total)
        os.close(fd)
        mapped = torch.from_file(path, shared=True, size=total, dtype=torch.uint8)
    finally:
        os.unlink(path)  # the mapping keeps the file alive until the last tensor over it is gone
    wrote_from = None
    for k, out_dtype, offset, nbytes in layout:
        v = state_dict[k]
        dest = mapped[offset:offset + nbytes].view(out_dtype).view(v.shape)
        if isinstance(v, NF4Tensor):
            if v.quantized_data.is_cuda:
                stage = _staging_buffer(v.numel(), v.dtype)
                v.get_original_weight(out=stage)
                wrote_from = v.quantized_data.device
                torch.cuda.current_stream(wrote_from).synchronize()
                dest.view(-1).copy_(stage)  # also the cast when dtype differs from the weight's own
            else:
                dest.copy_(v.to(dtype))
        else:
            dest.copy_(v.detach())
        state_dict[k] = dest


def _register_reparametrize_state_dict_hooks(
    module: nn.Module, dtype: torch.dtype = torch.bfloat16, offload_to_cpu: bool = True
) -> None:
    """Register the hook that strips NF4 from ``module.state_dict()``: the low-host-RAM one when ``_use_low_cpu_ram``
    is set, the ordinary one otherwise (``torchtune/modules/common_utils.py:206-237``)."""
    if _use_low_cpu_ram:
        if sys.platform == "win32":
            raise RuntimeError("Low RAM reparametrize_as_dtype_state_dict_post_hook is not supported on Windows.")
        hook = _low_ram_reparametrize_as_dtype_state_dict_post_hook
    else:
        hook = reparametrize_as_dtype_state_dict_post_hook
    module._register_state_dict_hook(partial(hook, dtype=dtype, offload_to_cpu=offload_to_cpu))
