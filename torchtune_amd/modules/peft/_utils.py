"""The small part of the adapter bookkeeping that callers of ``LoRALinear`` need
(``torchtune/modules/peft/_utils.py:19-83``): the ``AdapterModule`` protocol and the helpers that pick out and
freeze parameters by it."""
from __future__ import annotations

from typing import Dict, List, Protocol

from torch import nn


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
