"""Convolution samplers on the HIP kernels (mirror of opacus/grad_sample/conv.py).

Conv2d runs the implicit-im2col MFMA kernel; Conv1d is the same kernel on a height-one
image, as the reference's Conv1d branch does with ``unsqueeze(-2)`` (conv.py:71-88).
Conv3d runs the same kernel with a depth dimension in the gather (conv.py:89-96).
"""

from __future__ import annotations

from typing import Dict, List, Tuple, Union

import torch
import torch.nn as nn

from .. import kernels
from ._common import tag_sumsq
from .grad_sample_module import fused_scale, owns_output
from .utils import register_grad_sampler


def _pads(padding, kernel: int, dilation: int) -> Tuple[int, int]:
    """(before, after) padding of one dimension; "same" puts the smaller half first
    (opacus/utils/tensor_utils.py:128-134)."""
    if padding == "same":
        total = dilation * (kernel - 1)
        return total // 2, total - total // 2
    if padding == "valid":
        return 0, 0
    return int(padding), int(padding)


@register_grad_sampler([nn.Conv1d, nn.Conv2d, nn.Conv3d])
@owns_output
@fused_scale
def compute_conv_grad_sample(
    layer: Union[nn.Conv1d, nn.Conv2d, nn.Conv3d], activations: List[torch.Tensor], backprops: torch.Tensor, scale: float = 1.0
) -> Dict[nn.Parameter, torch.Tensor]:
    """Per-sample gradients ``[n, *weight.shape]`` and ``[n, out_channels]`` (conv.py:28-119).
    An empty batch yields zeros with a batch dimension of one (conv.py:46-53)."""
    x = activations[0]
    n = x.shape[0]
    want_b = layer.bias is not None and layer.bias.requires_grad
    ret = {}
    if n == 0:
        ret[layer.weight] = torch.zeros_like(layer.weight).unsqueeze(0)
        if want_b:
            ret[layer.bias] = torch.zeros_like(layer.bias).unsqueeze(0)
        return ret
    pad_is_str = isinstance(layer.padding, str)
    if isinstance(layer, nn.Conv3d):
        ksize, stride, dilation = tuple(layer.kernel_size), tuple(layer.stride), tuple(layer.dilation)
        pads3 = tuple(
            _pads(layer.padding if pad_is_str else layer.padding[d], ksize[d], dilation[d]) for d in range(3)
        )
        if layer.weight.requires_grad:
            gs, sumsq = kernels.conv3d_grad_sample(x, backprops, ksize, stride, pads3, dilation, layer.groups, scale=scale)
            ret[layer.weight] = tag_sumsq(gs.view(n, *layer.weight.shape), sumsq)
        if want_b:
            ret[layer.bias] = kernels.conv_bias_grad_sample(backprops, scale=scale)
        return ret
    if isinstance(layer, nn.Conv1d):
        x = x.unsqueeze(-2)
        b4 = backprops.unsqueeze(-2)
        ksize, stride, dilation = (1, layer.kernel_size[0]), (1, layer.stride[0]), (1, layer.dilation[0])
        pw = _pads(layer.padding if pad_is_str else layer.padding[0], ksize[1], dilation[1])
        pads = (0, 0, *pw)
    else:
        b4 = backprops
        ksize, stride, dilation = tuple(layer.kernel_size), tuple(layer.stride), tuple(layer.dilation)
        ph = _pads(layer.padding if pad_is_str else layer.padding[0], ksize[0], dilation[0])
        pw = _pads(layer.padding if pad_is_str else layer.padding[1], ksize[1], dilation[1])
        pads = (*ph, *pw)
    if layer.weight.requires_grad:
        gs, sumsq = kernels.conv2d_grad_sample(x, b4, ksize, stride, pads, dilation, layer.groups, scale=scale)
        ret[layer.weight] = tag_sumsq(gs.view(n, *layer.weight.shape), sumsq)
    if want_b:
        ret[layer.bias] = kernels.conv_bias_grad_sample(backprops, scale=scale)
    return ret
