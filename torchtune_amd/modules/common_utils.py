"""State-dict hooks that strip NF4 from checkpoints: every ``NF4Tensor`` in ``module.state_dict()`` is replaced
by its dequantised dense tensor, optionally moved to the CPU.  Same contract as
``reparametrize_as_dtype_state_dict_post_hook`` / ``_register_reparametrize_state_dict_hooks`` in the reference
(``torchtune/modules/common_utils.py:24-59,206-237``); the dequantisation is the HIP kernel."""
from __future__ import annotations

from functools import partial
from typing import Any, Dict

import torch
from torch import nn

from ..nf4_tensor import NF4Tensor


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


def _register_reparametrize_state_dict_hooks(
    module: nn.Module, dtype: torch.dtype = torch.bfloat16, offload_to_cpu: bool = True
) -> None:
    module._register_state_dict_hook(
        partial(reparametrize_as_dtype_state_dict_post_hook, dtype=dtype, offload_to_cpu=offload_to_cpu)
    )
