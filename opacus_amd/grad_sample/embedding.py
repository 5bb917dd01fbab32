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
