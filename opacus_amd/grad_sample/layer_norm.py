"""nn.LayerNorm sampler on the HIP kernel (mirror of opacus/grad_sample/layer_norm.py)."""

from __future__ import annotations

import math
from typing import Dict, List

import torch
import torch.nn as nn

from .. import kernels
from ._common import tag_sumsq
from .grad_sample_module import fused_scale, owns_output
from .utils import register_grad_sampler


@register_grad_sampler(nn.LayerNorm)
@owns_output
@fused_scale
def compute_layer_norm_grad_sample(
    layer: nn.LayerNorm, activations: List[torch.Tensor], backprops: torch.Tensor, scale: float = 1.0
) -> Dict[nn.Parameter, torch.Tensor]:
    """``layer_norm(x) * b`` for the weight and ``b`` for the bias, summed over all but the batch
    and the normalised dimensions (layer_norm.py:27-52). The normalisation is redone without
    affine, in registers."""
    want_w = layer.weight is not None and layer.weight.requires_grad
    want_b = layer.bias is not None and layer.bias.requires_grad
    ret = {}
    if not (want_w or want_b):
        return ret
    x = activations[0]
    numel = math.prod(layer.normalized_shape)
    gw, gb = kernels.layer_norm_grad_sample(
        x, backprops, numel, layer.eps, scale=scale, want_weight=want_w, want_bias=want_b
    )
    if want_w:
        ret[layer.weight] = tag_sumsq(gw.view(x.shape[0], *layer.normalized_shape), getattr(gw, "_dpk_sumsq", None))
    if want_b:
        ret[layer.bias] = tag_sumsq(gb.view(x.shape[0], *layer.normalized_shape), getattr(gb, "_dpk_sumsq", None))
    return ret
