"""nn.GroupNorm sampler on the HIP kernel (mirror of opacus/grad_sample/group_norm.py)."""

from __future__ import annotations

from typing import Dict, List

import torch
import torch.nn as nn

from .. import kernels
from .grad_sample_module import fused_scale, owns_output
from .utils import register_grad_sampler


@register_grad_sampler(nn.GroupNorm)
@owns_output
@fused_scale
def compute_group_norm_grad_sample(
    layer: nn.GroupNorm, activations: List[torch.Tensor], backprops: torch.Tensor, scale: float = 1.0
) -> Dict[nn.Parameter, torch.Tensor]:
    """``sum_spatial group_norm(x) * b`` for the weight and ``sum_spatial b`` for the bias,
    both ``[n, C]`` (group_norm.py:26-47). The normalisation is redone without affine."""
    want_w = layer.weight is not None and layer.weight.requires_grad
    want_b = layer.bias is not None and layer.bias.requires_grad
    ret = {}
    if not (want_w or want_b):
        return ret
    gw, gb = kernels.group_norm_grad_sample(
        activations[0], backprops, layer.num_groups, layer.eps, scale=scale, want_weight=want_w, want_bias=want_b
    )
    if want_w:
        ret[layer.weight] = gw
    if want_b:
        ret[layer.bias] = gb
    return ret
