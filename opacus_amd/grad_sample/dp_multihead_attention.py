"""Sampler of ``SequenceBias``, the key/value bias of DPMultiheadAttention
(mirror of opacus/grad_sample/dp_multihead_attention.py)."""

from __future__ import annotations

from typing import Dict, List

import torch
import torch.nn as nn

from ..layers.dp_multihead_attention import SequenceBias
from .utils import register_grad_sampler


@register_grad_sampler(SequenceBias)
def compute_sequence_bias_grad_sample(
    layer: SequenceBias, activations: List[torch.Tensor], backprops: torch.Tensor
) -> Dict[nn.Parameter, torch.Tensor]:
    """The bias is the last element of the output sequence, so its per-sample gradient is
    the backprop of that element (dp_multihead_attention.py:26-41): a slice, no arithmetic."""
    ret = {}
    if layer.bias.requires_grad:
        ret[layer.bias] = backprops[:, -1].contiguous()
    return ret
