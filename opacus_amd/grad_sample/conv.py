"""Convolution samplers on the HIP kernels (mirror of opacus/grad_sample/conv.py).

Conv2d runs the implicit-im2col MFMA kernel; Conv1d is the same kernel on a height-one
image, as the reference's Conv1d branch does with ``unsqueeze(-2)`` (conv.py:71-88).
Conv3d runs the same kernel with a depth dimension in the gather (conv.py:89-96).
"""

from __future__ import annotations

from typing import Dict, List, Tuple, Union

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import kernels
from ._common import tag_sumsq
from .grad_sample_module import fused_scale, owns_output
from .utils import register_grad_sampler, register_norm_sampler


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


def _conv2d_geometry(layer: Union[nn.Conv1d, nn.Conv2d], x: torch.Tensor, backprops: torch.Tensor):
    """Input, backprops, kernel, stride, (top, bottom, left, right) padding and dilation of a
    Conv1d (as a height-one image, conv.py:71-88) or Conv2d layer."""
    pad_is_str = isinstance(layer.padding, str)
    if isinstance(layer, nn.Conv1d):
        x, b4 = x.unsqueeze(-2), backprops.unsqueeze(-2)
        ksize, stride, dilation = (1, layer.kernel_size[0]), (1, layer.stride[0]), (1, layer.dilation[0])
        pads = (0, 0, *_pads(layer.padding if pad_is_str else layer.padding[0], ksize[1], dilation[1]))
    else:
        b4 = backprops
        ksize, stride, dilation = tuple(layer.kernel_size), tuple(layer.stride), tuple(layer.dilation)
        ph = _pads(layer.padding if pad_is_str else layer.padding[0], ksize[0], dilation[0])
        pw = _pads(layer.padding if pad_is_str else layer.padding[1], ksize[1], dilation[1])
        pads = (*ph, *pw)
    return x, b4, ksize, stride, pads, dilation


@register_norm_sampler([nn.Conv1d, nn.Conv2d])
@fused_scale
def compute_conv_norm_sample(
    layer: Union[nn.Conv1d, nn.Conv2d], activations: List[torch.Tensor], backprops: torch.Tensor, scale: float = 1.0
) -> Dict[nn.Parameter, torch.Tensor]:
    """Per-sample gradient norms of a convolution without storing the per-sample gradients.

    The reference has no norm sampler for convolutions: under fast gradient clipping it forms
    every per-sample gradient, norms it and drops it
    (grad_sample_module_fast_gradient_clipping.py:226-250). Two routes here, by cost. With q
    output positions, p kernel elements and O output channels per sample, the gradient is the
    contraction ``b[O, q] U[p, q]^T``, the same algebra as a Linear layer over a sequence of q
    positions (conv.py:102), so its norm is also ``sum_{q,q'} (b_q . b_q')(U_q . U_q')``
    (linear.py:83-89): for few positions (the late layers of a CNN) the Gram route on the
    unfolded input costs ``q^2 (O + p)`` against ``q O p``. Otherwise the convolution kernel
    forms the gradient tiles and squares them in its epilogue, never storing them."""
    x = activations[0]
    n = x.shape[0]
    want_w = layer.weight.requires_grad
    want_b = layer.bias is not None and layer.bias.requires_grad
    ret = {}
    if n == 0:
        empty = torch.zeros((0,), device=backprops.device, dtype=torch.float32)
        if want_w:
            ret[layer.weight] = empty
        if want_b:
            ret[layer.bias] = empty.clone()
        return ret
    if want_w:
        x4, b4, ksize, stride, pads, dilation = _conv2d_geometry(layer, x, backprops)
        O, q = b4.shape[1], b4.shape[2] * b4.shape[3]
        p = (x4.shape[1] // layer.groups) * ksize[0] * ksize[1]
        gram, direct = 0.6 * q * q * (O + p), float(q) * O * p  # 0.6: the tile pairs on and above the diagonal
        if layer.groups == 1 and q > 1 and gram < 0.5 * direct:
            xp = x4.to(b4.dtype)
            if pads[0] != pads[1] or pads[2] != pads[3]:
                xp, sym = F.pad(xp, (pads[2], pads[3], pads[0], pads[1])), (0, 0)
            else:
                sym = (pads[0], pads[2])
            unfolded = F.unfold(xp, kernel_size=ksize, dilation=dilation, padding=sym, stride=stride)  # [n, p, q]
            nw, _ = kernels.linear_ghost_norm(
                b4.flatten(2).transpose(1, 2), unfolded.transpose(1, 2), scale=scale, want_weight=True, want_bias=False
            )
        else:
            _, sumsq = kernels.conv2d_grad_sample(x4, b4, ksize, stride, pads, dilation, layer.groups, scale=scale, norm_only=True)
            nw = sumsq.sqrt_()
        ret[layer.weight] = nw
    if want_b:
        gs_b = kernels.conv_bias_grad_sample(backprops, scale=scale)
        ret[layer.bias] = gs_b._dpk_sumsq.sqrt()
    return ret


compute_conv_norm_sample.reference_materialises = True
