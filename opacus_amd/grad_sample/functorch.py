"""Generic per-sample gradients for layers without a registered sampler.

Mirror of opacus/grad_sample/functorch.py: the layer is re-run functionally on one
sample at a time under ``torch.func.vmap(grad(...))``. This is plain PyTorch on the
tensors' own device, outside the HIP hot path; it exists so that a model with an
unsupported layer still trains.
"""

from __future__ import annotations

import copy
from contextlib import nullcontext

import torch
import torch.nn as nn
from torch.func import functional_call, grad, vmap


def make_functional(mod: nn.Module, disable_autograd_tracking: bool = False):
    """``(fmodel, params)`` with ``fmodel(params, *args)`` calling a stateless copy of ``mod``."""
    named = dict(mod.named_parameters())
    names = tuple(named.keys())
    values = tuple(named.values())
    skeleton = copy.deepcopy(mod)
    skeleton.to("meta")
    if hasattr(skeleton, "allow_grad_accumulation"):
        skeleton.allow_grad_accumulation()

    def fmodel(new_values, *args, **kwargs):
        return functional_call(skeleton, dict(zip(names, new_values)), args, kwargs)

    if disable_autograd_tracking:
        values = tuple(v.detach() for v in values)
    return fmodel, values


def prepare_layer(layer: nn.Module, batch_first: bool = True) -> None:
    """Attaches ``layer.ft_compute_sample_grad`` (opacus/grad_sample/functorch.py:58-105)."""
    if len(list(layer.buffers())) > 0:
        raise NotImplementedError("This layer has buffers and is not supported by Opacus")
    if type(layer) is nn.EmbeddingBag:
        raise NotImplementedError("Functorch does not support EmbeddingBag yet")
    flayer, _ = make_functional(layer)
    batch_dim = 0 if batch_first else 1

    def loss_of_one_sample(params, activations, backprops):
        a = activations.unsqueeze(batch_dim)
        b = backprops.unsqueeze(batch_dim)
        mixed = activations.dtype != params[0].dtype
        ctx = torch.amp.autocast(device_type=activations.device.type, dtype=activations.dtype) if mixed else nullcontext()
        with ctx:
            return (flayer(params, a) * b).sum()

    layer.ft_compute_sample_grad = vmap(grad(loss_of_one_sample), in_dims=(None, 0, 0))


def ft_compute_per_sample_gradient(layer: nn.Module, activations, backprops: torch.Tensor):
    """``{param: grad_sample}`` for all parameters of ``layer`` (functorch.py:108-129)."""
    parameters = list(layer.parameters(recurse=True))
    if not hasattr(layer, "ft_compute_sample_grad"):
        prepare_layer(layer)
    a = activations[0]
    if a.dtype != backprops.dtype and a.is_floating_point():
        a = a.to(backprops.dtype)
    per_sample = layer.ft_compute_sample_grad(parameters, a, backprops)
    return {p: per_sample[i] for i, p in enumerate(parameters)}
