"""Sampler registry and module wrapping (mirror of opacus/grad_sample/utils.py).

``register_grad_sampler`` / ``register_norm_sampler`` are the plugin boundary: a sampler
is ``fn(layer, activations, backprops) -> {parameter: tensor}`` where ``activations`` are
the detached forward inputs, ``backprops`` the detached output gradient, batch first and
already scaled to a sum-reduced loss. The last registration for a class wins.
"""

from __future__ import annotations

from typing import Sequence, Type, Union

import torch.nn as nn

from .grad_sample_module import GradSampleHooks, GradSampleModule
from .grad_sample_module_fast_gradient_clipping import (
    GradSampleHooksFastGradientClipping,
    GradSampleModuleFastGradientClipping,
)
from .gsm_base import AbstractGradSampleModule


def _as_list(target) -> Sequence[Type[nn.Module]]:
    return target if isinstance(target, Sequence) else [target]


def register_grad_sampler(target_class_or_classes: Union[Type[nn.Module], Sequence[Type[nn.Module]]]):
    """Decorator: use the function as per-sample-gradient sampler of the given layer class(es)
    in both the hooks and the fast-gradient-clipping engines (grad_sample/utils.py:37-63)."""

    def decorator(f):
        for cls in _as_list(target_class_or_classes):
            GradSampleHooks.GRAD_SAMPLERS[cls] = f
            GradSampleHooksFastGradientClipping.GRAD_SAMPLERS[cls] = f
        return f

    return decorator


def register_norm_sampler(target_class_or_classes: Union[Type[nn.Module], Sequence[Type[nn.Module]]]):
    """Decorator: use the function as ghost-clipping norm sampler of the given layer class(es)
    (grad_sample/utils.py:66-89)."""

    def decorator(f):
        for cls in _as_list(target_class_or_classes):
            GradSampleHooksFastGradientClipping.NORM_SAMPLERS[cls] = f
        return f

    return decorator


_MODULE_CLASSES = {
    "hooks": GradSampleModule,
    "functorch": GradSampleModule,
    "ghost": GradSampleModuleFastGradientClipping,
}
_HOOKS_CLASSES = {
    "hooks": GradSampleHooks,
    "functorch": GradSampleHooks,
    "ghost": GradSampleHooksFastGradientClipping,
}
_NOT_BUILT = ("ew", "ghost_fsdp", "ghost_tp", "no_op")


def _lookup(table, grad_sample_mode: str):
    if grad_sample_mode in table:
        return table[grad_sample_mode]
    if grad_sample_mode in _NOT_BUILT:
        raise NotImplementedError(
            f"grad_sample_mode={grad_sample_mode!r} is outside this build: only the hooks-based paths "
            f"{list(table.keys())} run on the HIP kernels"
        )
    raise ValueError(f"Unexpected grad_sample_mode: {grad_sample_mode}. Allowed values: {list(table.keys())}")


def get_gsm_class(grad_sample_mode: str) -> Type[AbstractGradSampleModule]:
    """Wrapper class for a ``grad_sample_mode`` (grad_sample/utils.py:136-158)."""
    return _lookup(_MODULE_CLASSES, grad_sample_mode)


def get_hooks_class(grad_sample_mode: str):
    """Hooks (non-wrapping) class for a ``grad_sample_mode`` (grad_sample/utils.py:161-183)."""
    return _lookup(_HOOKS_CLASSES, grad_sample_mode)


def prepare_module(model: nn.Module, grad_sample_mode: str, wrap_model: bool = True, *args, **kwargs):
    """Wraps the model, or with ``wrap_model=False`` attaches a hooks object to it and
    returns that (grad_sample/utils.py:92-119)."""
    cls = get_gsm_class(grad_sample_mode) if wrap_model else get_hooks_class(grad_sample_mode)
    if grad_sample_mode == "functorch":
        kwargs["force_functorch"] = True
    return cls(model, *args, **kwargs)


def wrap_model(model: nn.Module, grad_sample_mode: str, *args, **kwargs) -> AbstractGradSampleModule:
    """Kept for callers of the older name (grad_sample/utils.py:122-133)."""
    return prepare_module(model, grad_sample_mode, True, *args, **kwargs)
