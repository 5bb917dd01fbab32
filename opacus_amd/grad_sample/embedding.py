"""nn.Embedding samplers on the HIP kernels (mirror of opacus/grad_sample/embedding.py and
opacus/grad_sample/embedding_norm_sample.py)."""

from __future__ import annotations

from typing import Dict, List

import torch
import torch.nn as nn

from .. import kernels
from .grad_sample_module import fused_scale, owns_output
from .utils import register_grad_sampler, register_norm_sampler


@register_grad_sampler(nn.Embedding)
@owns_output
@fused_scale
def compute_embedding_grad_sample(
    layer: nn.Embedding, activations: List[torch.Tensor], backprops: torch.Tensor, scale: float = 1.0
) -> Dict[nn.Parameter, torch.Tensor]:
    """Per-sample gradient ``[n, num_embeddings, dim]``: backprop rows summed per id
    (embedding.py:25-64). ``padding_idx`` is not special-cased, as in the reference; an
    empty batch yields zeros with a batch dimension of one (:44-46)."""
    ids = activations[0]
    ret = {}
    if layer.weight.requires_grad:
        if ids.shape[0] == 0:
            ret[layer.weight] = torch.zeros_like(layer.weight).unsqueeze(0)
            return ret
        ret[layer.weight] = kernels.embedding_grad_sample(ids, backprops, layer.num_embeddings, scale=scale)
    return ret


@register_grad_sampler(nn.EmbeddingBag)
@owns_output
@fused_scale
def compute_embeddingbag_gradsampler(
    layer: nn.EmbeddingBag, activations: List[torch.Tensor], backprops: torch.Tensor, scale: float = 1.0
) -> Dict[nn.Parameter, torch.Tensor]:
    """Per-sample gradient ``[bags, num_embeddings, dim]`` (embedding.py:67-94): every index of
    bag ``i`` receives ``backprops[i]`` (divided by the bag length for ``mode="mean"``); an index
    repeated inside a bag receives it once, ``per_sample_weights`` and ``padding_idx`` are not
    looked at - all as in the reference. A 2-D index tensor without offsets is one bag per row."""
    if not layer.weight.requires_grad:
        return {}
    index = activations[0]
    if len(activations) > 1 and activations[1] is not None:
        offsets = activations[1]
    elif index.dim() == 2:
        offsets = torch.arange(0, index.numel(), index.shape[1], device=index.device, dtype=torch.int64)
    else:
        raise ValueError("EmbeddingBag needs offsets for a 1-D index tensor")
    gs = kernels.embedding_bag_grad_sample(index, offsets, backprops, layer.num_embeddings, mode=layer.mode, scale=scale)
    return {layer.weight: gs}


@register_norm_sampler(nn.Embedding)
@fused_scale
def compute_embedding_norm_sample(
    layer: nn.Embedding, activations: List[torch.Tensor], backprops: torch.Tensor, scale: float = 1.0
) -> Dict[nn.Parameter, torch.Tensor]:
    """Per-sample gradient norm of the embedding table without the ``[n, V, dim]`` tensor:
    rows that share (sample, id) are summed, squared and added up per sample
    (embedding_norm_sample.py:27-151)."""
    if not layer.weight.requires_grad:
        return {}
    return {layer.weight: kernels.embedding_ghost_norm(activations[0], backprops, scale=scale)}
