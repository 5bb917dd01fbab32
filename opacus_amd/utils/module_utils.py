"""Small traversal helpers over ``nn.Module`` trees (opacus/utils/module_utils.py)."""

from __future__ import annotations

from typing import Iterable, List, Tuple

import torch.nn as nn


def has_trainable_params(module: nn.Module) -> bool:
    """True if the module itself (not its children) owns a parameter that requires grad."""
    return any(p is not None and p.requires_grad for p in module._parameters.values())


def requires_grad(module: nn.Module, *, recurse: bool = False) -> bool:
    """True if any parameter of the module (its own only, unless ``recurse``) requires grad."""
    if not recurse:
        return any(p is not None and p.requires_grad for p in module._parameters.values())
    return any(p.requires_grad for p in module.parameters(recurse))


def trainable_parameters(module: nn.Module) -> Iterable[Tuple[str, nn.Parameter]]:
    """``(name, parameter)`` for every parameter of the tree that requires grad."""
    return ((name, p) for name, p in module.named_parameters() if p.requires_grad)


def trainable_parameter_list(module: nn.Module) -> List[nn.Parameter]:
    """The parameters of the tree that require grad. The hooks call this several times per
    layer and step, so a module without children reads its own table directly."""
    if not module._modules:
        seen, out = set(), []
        for p in module._parameters.values():
            if p is not None and p.requires_grad and id(p) not in seen:
                seen.add(id(p))
                out.append(p)
        return out
    return [p for _, p in trainable_parameters(module)]


def trainable_modules(module: nn.Module) -> Iterable[Tuple[str, nn.Module]]:
    """``(name, submodule)`` for every submodule that owns a trainable parameter itself."""
    return ((name, m) for name, m in module.named_modules() if has_trainable_params(m))
