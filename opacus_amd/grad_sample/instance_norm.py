"""nn.InstanceNorm{1,2,3}d sampler (mirror of opacus/grad_sample/instance_norm.py).

Instance normalisation is group normalisation with one channel per group, so it runs on the
GroupNorm kernel with ``groups == C``.
"""

from __future__ import annotations

from typing import Dict, List, Union

import torch
import torch.nn as nn

from .. import kernels
from .grad_sample_module import fused_scale, owns_output
from .utils import register_grad_sampler


@register_grad_sampler([nn.InstanceNorm1d, nn.InstanceNorm2d, nn.InstanceNorm3d])
@owns_output
@fused_scale
def compute_instance_norm_grad_sample(
    layer: Union[nn.InstanceNorm1d, nn.InstanceNorm2d, nn.InstanceNorm3d],
    activations: List[torch.Tensor],
    backprops: torch.Tensor,
    scale: float = 1.0,
) -> Dict[nn.Parameter, torch.Tensor]:
    """``sum_spatial instance_norm(x) * b`` and ``sum_spatial b``, both ``[n, C]``
    (instance_norm.py:30-56)."""
    want_w = layer.weight is not None and layer.weight.requires_grad
    want_b = layer.bias is not None and layer.bias.requires_grad
    ret = {}
    if not (want_w or want_b):
        return ret
    x = activations[0]
    gw, gb = kernels.group_norm_grad_sample(
        x, backprops, x.shape[1], layer.eps, scale=scale, want_weight=want_w, want_bias=want_b
    )
    if want_w:
        ret[layer.weight] = gw
    if want_b:
        ret[layer.bias] = gb
    return ret
