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


def reparametrize_as_dtype_state_dict_post_hook(
    model: nn.Module,
    state_dict: Dict[str, Any],
    *args: Any,
    dtype: torch.dtype = torch.bfloat16,
    offload_to_cpu: bool = True,
    **kwargs: Any,
) -> None:
    """State-dict post hook: NF4 entries become dense ``dtype`` tensors (on the CPU if ``offload_to_cpu``)."""
    for k, v in state_dict.items():
        if isinstance(v, NF4Tensor):
            dense = v.to(dtype)
            state_dict[k] = dense.cpu() if offload_to_cpu else dense


def _register_reparametrize_state_dict_hooks(
    module: nn.Module, dtype: torch.dtype = torch.bfloat16, offload_to_cpu: bool = True
) -> None:
    module._register_state_dict_hook(
        partial(reparametrize_as_dtype_state_dict_post_hook, dtype=dtype, offload_to_cpu=offload_to_cpu)
    )
