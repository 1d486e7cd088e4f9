"""The part of the adapter bookkeeping that callers of ``LoRALinear`` need
(``torchtune/modules/peft/_utils.py:19-83,115-133,193-321``): the ``AdapterModule`` protocol, the helpers that pick
out and freeze parameters by it, the adapter part of a state dict, the switch that runs a model without its adapters,
and the merge of the adapters into the base weights for a checkpoint."""
from __future__ import annotations

import contextlib
from typing import Any, Dict, Generator, List, Optional, Protocol, Set

import torch
from torch import nn

from ... import ops
from ...nf4_tensor import NF4Tensor


class AdapterModule(Protocol):
    """An ``nn.Module`` that owns adapter weights names them through ``adapter_params``."""

    def adapter_params(self) -> List[str]:
        ...


def get_adapter_params(model: nn.Module) -> Dict[str, nn.Parameter]:
    """All parameters that some module of ``model`` declares as adapter parameters, keyed by full name."""
    found: Dict[str, nn.Parameter] = {}
    for mod_name, mod in model.named_modules():
        names = getattr(mod, "adapter_params", None)
        if not callable(names):
            continue
        wanted = set(names())
        for pname, p in mod.named_parameters(recurse=True):
            if pname in wanted:
                found[f"{mod_name}.{pname}" if mod_name else pname] = p
                wanted.discard(pname)
        assert not wanted, f"Adapter params {wanted} not converted"
    return found


def set_trainable_params(model: nn.Module, adapter_params: Dict[str, nn.Parameter]) -> None:
    """Freeze everything except the given parameters."""
    for name, p in model.named_parameters():
        p.requires_grad_(name in adapter_params)


def get_adapter_state_dict(state_dict: Dict[str, Any], device: Optional[str] = "cpu") -> Dict[str, Any]:
    """The adapter entries of an unsharded model state dict (keys that contain ``lora`` or ``magnitude``), moved to
    ``device`` (``torchtune/modules/peft/_utils.py:115-133``)."""
    return {k: v.to(device) for k, v in state_dict.items() if "lora" in k or "magnitude" in k}


def _adapter_switches(model: nn.Module):
    for _, mod in model.named_modules():
        if callable(getattr(mod, "adapter_params", None)) and hasattr(mod, "disabled"):
            yield mod


@contextlib.contextmanager
def disable_adapter(model: nn.Module) -> Generator[None, None, None]:
    """Run ``model`` as its base model: every module that declares adapter parameters and has a ``disabled`` flag
    skips its adapter inside the ``with`` block and gets it back afterwards, also when the block raises
    (``torchtune/modules/peft/_utils.py:274-321``; DPO uses it to get the reference model out of the policy)."""
    for mod in _adapter_switches(model):
        mod.disabled = True
    try:
        yield
    finally:
        for mod in _adapter_switches(model):
            mod.disabled = False


def _get_lora_modules(state_dict: Dict[str, Any]) -> Set[str]:
    """Module prefixes that own a ``lora_a.weight`` / ``lora_b.weight`` pair in ``state_dict``."""
    return {k[: -len(".lora_a.weight")] for k in state_dict if k.endswith(".lora_a.weight")}


@torch.no_grad()
def get_merged_lora_ckpt(state_dict: Dict[str, Any], rank: int, alpha: float, use_distributed_barriers: bool = False, *,
                         offload_to_cpu: bool = False) -> Dict[str, Any]:
    """Fold every LoRA pair of ``state_dict`` into its base weight and delete the adapter entries; modifies and
    returns ``state_dict`` (``torchtune/modules/peft/_utils.py:193-271``; MoE experts raise).

    Plain LoRA: ``W += (alpha / rank) * B @ A``.  With a DoRA ``magnitude`` entry the merged weight is
    ``(W + (alpha / rank) * B @ A) * (magnitude / ||W + (alpha / rank) * B @ A||_row)`` and the magnitude is deleted too.

    A base weight that is still an ``NF4Tensor`` on the GPU (a state dict taken without the dequantising hook) is
    dequantised and merged in one pass by the HIP kernel; a dense weight is updated as the reference does.
    ``use_distributed_barriers`` is the reference's fourth parameter (its checkpoint client passes it by keyword,
    ``torchtune/training/checkpointing/_checkpoint_client.py:177-182``); there is one process per GPU and no barrier to
    take here, so it is accepted and ignored.  ``offload_to_cpu`` (keyword only, not in the reference's signature) makes
    that kernel store the merged weight of a plain LoRA module straight into pinned host memory, so the dense merged
    weight never exists on the GPU.
    """
    wrote_to_host = None
    scale = alpha / rank
    for module in sorted(_get_lora_modules(state_dict)):
        if "experts" in module:
            raise NotImplementedError(f"{module}: merging MoE experts is not part of this build")
        a = state_dict[f"{module}.lora_a.weight"]
        b = state_dict[f"{module}.lora_b.weight"]
        w = state_dict[f"{module}.weight"]
        magnitude = state_dict.get(f"{module}.magnitude", None)
        fused = (
            isinstance(w, NF4Tensor) and w.is_cuda and w.block_size == 64 and w.dtype == torch.bfloat16
            and a.dtype == torch.bfloat16 and b.dtype == torch.bfloat16 and a.shape[0] % 8 == 0 and 0 < a.shape[0] <= 64
        )
        if fused:
            N, K = w.shape
            host = None
            if offload_to_cpu and magnitude is None:
                host = torch.empty(N, K, dtype=torch.bfloat16, pin_memory=True)
                wrote_to_host = w.device
            merged = ops.nf4_dequantize_merge(w.quantized_data, w.block_scalers(), N, K, a.to(w.device), b.to(w.device), scale,
                                              out=host)
        elif magnitude is not None or isinstance(w, NF4Tensor):
            merged = w.to(a.dtype) + scale * b @ a
        else:
            w += scale * b @ a
            merged = w
        if magnitude is not None:
            weight_norm = torch.linalg.norm(merged, dim=1)
            merged *= (magnitude.to(merged.device) / weight_norm).view(-1, 1)
            del state_dict[f"{module}.magnitude"]
        if offload_to_cpu and merged.is_cuda:
            merged = merged.cpu()
        state_dict[f"{module}.weight"] = merged
        del state_dict[f"{module}.lora_a.weight"]
        del state_dict[f"{module}.lora_b.weight"]
    if wrote_to_host is not None:
        torch.cuda.current_stream(wrote_to_host).synchronize()
    return state_dict
