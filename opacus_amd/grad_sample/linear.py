"""nn.Linear samplers on the HIP kernels (mirror of opacus/grad_sample/linear.py)."""

from __future__ import annotations

from typing import Dict, List

import torch
import torch.nn as nn

from .. import kernels
from ._common import tag_sumsq
from .grad_sample_module import fused_scale, owns_output
from .utils import register_grad_sampler, register_norm_sampler


@register_grad_sampler(nn.Linear)
@owns_output
@fused_scale
def compute_linear_grad_sample(
    layer: nn.Linear, activations: List[torch.Tensor], backprops: torch.Tensor, scale: float = 1.0
) -> Dict[nn.Parameter, torch.Tensor]:
    """Per-sample gradients of ``nn.Linear`` (linear.py:29-51): weight ``[n, out, in]`` summed
    over every middle dimension, bias ``[n, out]``."""
    a = activations[0]
    ret = {}
    if layer.weight.requires_grad:
        gs, sumsq = kernels.linear_grad_sample(backprops, a, scale=scale)
        ret[layer.weight] = tag_sumsq(gs, sumsq)
    if layer.bias is not None and layer.bias.requires_grad:
        ret[layer.bias] = kernels.linear_bias_grad_sample(backprops, scale=scale)
    return ret


@register_norm_sampler(nn.Linear)
@fused_scale
def compute_linear_norm_sample(
    layer: nn.Linear, activations: List[torch.Tensor], backprops: torch.Tensor, scale: float = 1.0
) -> Dict[nn.Parameter, torch.Tensor]:
    """Per-sample gradient norms of ``nn.Linear`` without the gradients (linear.py:54-93).

    2-d backprops use the rank-one closed form, 3-d the T x T Gram contraction. Backprops
    with more middle dimensions, for which the reference returns nothing, are treated as
    3-d with the middle dimensions flattened.
    """
    want_w = layer.weight.requires_grad
    want_b = layer.bias is not None and layer.bias.requires_grad
    ret = {}
    if not (want_w or want_b):
        return ret
    nw, nb = kernels.linear_ghost_norm(backprops, activations[0], scale=scale, want_weight=want_w, want_bias=want_b)
    if want_w:
        ret[layer.weight] = nw
    if want_b:
        ret[layer.bias] = nb
    return ret
