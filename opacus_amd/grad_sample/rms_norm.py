"""nn.RMSNorm sampler on the HIP kernel (mirror of opacus/grad_sample/rms_norm.py)."""

from __future__ import annotations

import math
from typing import Dict, List

import torch
import torch.nn as nn

from .. import kernels
from ._common import tag_sumsq
from .grad_sample_module import fused_scale, owns_output
from .utils import register_grad_sampler


@register_grad_sampler(nn.RMSNorm)
@owns_output
@fused_scale
def compute_rms_norm_grad_sample(
    layer: nn.RMSNorm, activations: List[torch.Tensor], backprops: torch.Tensor, scale: float = 1.0
) -> Dict[nn.Parameter, torch.Tensor]:
    """``rms_norm(x) * b`` summed over all but the batch and the normalised dimensions
    (rms_norm.py:27-47). ``eps=None`` means the input dtype's machine epsilon, as in
    ``torch.nn.functional.rms_norm``."""
    if layer.weight is None or not layer.weight.requires_grad:
        return {}
    x = activations[0]
    eps = layer.eps if layer.eps is not None else torch.finfo(x.dtype).eps
    numel = math.prod(layer.normalized_shape)
    gw = kernels.rms_norm_grad_sample(x, backprops, numel, eps, scale=scale)
    return {layer.weight: tag_sumsq(gw.view(x.shape[0], *layer.normalized_shape), gw._dpk_sumsq if x.shape[0] else None)}
