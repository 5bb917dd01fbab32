"""Multi-head attention built from ``nn.Linear`` so that per-sample gradients can be taken.

Mirror of opacus/layers/dp_multihead_attention.py: ``DPMultiheadAttention`` takes the
arguments of ``torch.nn.MultiheadAttention``, returns its outputs and exchanges state dicts
with it, but keeps its projections in four ``nn.Linear`` modules (``qlinear``, ``klinear``,
``vlinear``, ``out_proj``) and its optional key/value biases in two ``SequenceBias`` modules,
where the grad-sample hooks find them (torch's module calls ``F.multi_head_attention_forward``
on raw parameters, which no hook can see).

When the averaged attention weights are not asked for (``need_weights=False``) the
attention itself runs through ``F.scaled_dot_product_attention``, i.e. the fused attention
kernels of the GPU; otherwise the weights are formed explicitly, as they have to be returned.
"""

from __future__ import annotations

import warnings
from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor


class SequenceBias(nn.Module):
    """Appends one learned vector to the end of a sequence: ``[L, N, E] -> [L + 1, N, E]``, or
    ``[N, L, E] -> [N, L + 1, E]`` with ``batch_first`` (dp_multihead_attention.py:25-67)."""

    def __init__(self, embed_dim: int, batch_first: bool = False):
        super().__init__()
        self.batch_first = batch_first
        self.bias = nn.Parameter(torch.empty(embed_dim))
        self._reset_parameters()

    def _reset_parameters(self) -> None:
        nn.init.normal_(self.bias)

    def forward(self, x: Tensor) -> Tensor:
        if self.batch_first:
            return torch.cat([x, self.bias.expand(x.shape[0], 1, -1)], dim=1)
        return torch.cat([x, self.bias.expand(1, x.shape[1], -1)], dim=0)


def _torch_keys_to_ours(module: "DPMultiheadAttention", state_dict, prefix, *_):
    """Load pre-hook: accepts the keys of ``torch.nn.MultiheadAttention`` (:142-186)."""

    def move(src: str, dst: str, f=lambda t: t):
        if prefix + src in state_dict:
            state_dict[prefix + dst] = f(state_dict.pop(prefix + src))

    for kind in ("weight", "bias"):
        key = prefix + f"in_proj_{kind}"
        if key in state_dict:
            q, k, v = state_dict.pop(key).chunk(3, dim=0)
            state_dict[prefix + f"qlinear.{kind}"] = q
            state_dict[prefix + f"klinear.{kind}"] = k
            state_dict[prefix + f"vlinear.{kind}"] = v
    move("q_proj_weight", "qlinear.weight")
    move("k_proj_weight", "klinear.weight")
    move("v_proj_weight", "vlinear.weight")
    move("bias_k", "seq_bias_k.bias", lambda t: t.reshape(-1))
    move("bias_v", "seq_bias_v.bias", lambda t: t.reshape(-1))


def _ours_to_torch_keys(module: "DPMultiheadAttention", state_dict, prefix, _local_metadata):
    """State-dict hook: saves under the keys of ``torch.nn.MultiheadAttention`` (:334-400)."""

    def take(name: str):
        return state_dict.pop(prefix + name, None)

    qw, kw, vw = take("qlinear.weight"), take("klinear.weight"), take("vlinear.weight")
    if module.kdim == module.embed_dim and module.vdim == module.embed_dim:
        state_dict[prefix + "in_proj_weight"] = torch.cat((qw, kw, vw), dim=0)
    else:
        state_dict[prefix + "q_proj_weight"] = qw
        state_dict[prefix + "k_proj_weight"] = kw
        state_dict[prefix + "v_proj_weight"] = vw
    qb, kb, vb = take("qlinear.bias"), take("klinear.bias"), take("vlinear.bias")
    if qb is not None:
        state_dict[prefix + "in_proj_bias"] = torch.cat((qb, kb, vb), dim=0)
    bk, bv = take("seq_bias_k.bias"), take("seq_bias_v.bias")
    if bk is not None:
        state_dict[prefix + "bias_k"] = bk.reshape(1, 1, -1)
        state_dict[prefix + "bias_v"] = bv.reshape(1, 1, -1)
    # torch's key order: in_proj (or q/k/v_proj), biases, then out_proj
    for name in ("out_proj.weight", "out_proj.bias"):
        value = take(name)
        if value is not None:
            state_dict[prefix + name] = value
    return state_dict


class DPMultiheadAttention(nn.Module):
    """Drop-in replacement of ``torch.nn.MultiheadAttention`` for DP training
    (dp_multihead_attention.py:70-400). Batched (3-d) inputs only; no causal flag."""

    def __init__(
        self,
        embed_dim,
        num_heads,
        dropout=0.0,
        bias=True,
        add_bias_kv=False,
        add_zero_attn=False,
        kdim=None,
        vdim=None,
        batch_first=False,
        device=None,
        dtype=None,
    ):
        super().__init__()
        kw = {"device": device, "dtype": dtype}
        self.embed_dim = embed_dim
        self.kdim = kdim if kdim is not None else embed_dim
        self.vdim = vdim if vdim is not None else embed_dim
        # nn.TransformerEncoderLayer takes its fused fast path when this is true; that path
        # reads in_proj_weight directly and would bypass the Linear modules (:96-97)
        self._qkv_same_embed_dim = False
        self.num_heads = num_heads
        self.batch_first = batch_first
        self.head_dim = embed_dim // num_heads
        assert self.head_dim * num_heads == self.embed_dim, "embed_dim must be divisible by num_heads"

        self.qlinear = nn.Linear(embed_dim, embed_dim, bias=bias, **kw)
        self.klinear = nn.Linear(self.kdim, embed_dim, bias=bias, **kw)
        self.vlinear = nn.Linear(self.vdim, embed_dim, bias=bias, **kw)
        self.out_proj = nn.Linear(embed_dim, embed_dim, bias=bias, **kw)
        self.add_bias_kv = add_bias_kv
        if add_bias_kv:
            # in the caller's layout, so that the grad-sample hooks find the batch where they
            # find it for the Linear modules
            self.seq_bias_k = SequenceBias(embed_dim, batch_first=batch_first)
            self.seq_bias_v = SequenceBias(embed_dim, batch_first=batch_first)
            if device is not None or dtype is not None:
                self.seq_bias_k.to(**kw)
                self.seq_bias_v.to(**kw)
        self.add_zero_attn = add_zero_attn
        self.dropout = nn.Dropout(dropout)
        # read (and found absent) by nn.TransformerEncoderLayer.forward
        self.in_proj_weight = None
        self.in_proj_bias = None
        self._register_state_dict_hook(_ours_to_torch_keys)
        self.register_load_state_dict_pre_hook(_torch_keys_to_ours)

    def forward(
        self,
        query: Tensor,
        key: Tensor,
        value: Tensor,
        key_padding_mask: Optional[Tensor] = None,
        need_weights: bool = True,
        attn_mask: Optional[Tensor] = None,
        is_causal: bool = False,
    ) -> Tuple[Tensor, Optional[Tensor]]:
        assert query.dim() == 3, "The query must have a dimension of 3."
        assert not is_causal, "We currently do not support causal mask. Will fix it in the future."
        if self.batch_first:
            bsz, tgt_len, embed_dim = query.shape
        else:
            tgt_len, bsz, embed_dim = query.shape
        if embed_dim != self.embed_dim:
            raise ValueError(f"query has as size of {embed_dim} while the embedding size is {self.embed_dim}")
        H, hd = self.num_heads, self.head_dim

        q, k, v = self.qlinear(query), self.klinear(key), self.vlinear(value)
        if self.add_bias_kv:
            k, v = self.seq_bias_k(k), self.seq_bias_v(v)
        if self.batch_first:  # to [L, N, E], the layout of the masks and of torch's module
            q, k, v = (x.transpose(0, 1) for x in (q, k, v))

        if attn_mask is not None:
            if attn_mask.dtype == torch.uint8:
                warnings.warn("Byte tensor for attn_mask in nn.MultiheadAttention is deprecated. Use bool tensor instead.")
                attn_mask = attn_mask.to(torch.bool)
            elif attn_mask.dtype not in (torch.float32, torch.float64, torch.bool, q.dtype):
                raise ValueError(f"Only float, byte, and bool types are supported for attn_mask, not {attn_mask.dtype}.")
            keys = k.shape[0] - (1 if self.add_bias_kv else 0)  # the mask is given for the caller's keys
            if attn_mask.dim() == 2:
                if list(attn_mask.shape) != [tgt_len, keys]:
                    raise ValueError("The size of the 2D attn_mask is not correct.")
                attn_mask = attn_mask.unsqueeze(0)
            elif attn_mask.dim() == 3:
                if list(attn_mask.shape) != [bsz * H, tgt_len, keys]:
                    raise ValueError("The size of the 3D attn_mask is not correct.")
            else:
                raise ValueError(f"attn_mask's dimension {attn_mask.dim()} is not supported")
        if key_padding_mask is not None and key_padding_mask.dtype == torch.uint8:
            warnings.warn("Byte tensor for key_padding_mask in nn.MultiheadAttention is deprecated. Use bool tensor instead.")
            key_padding_mask = key_padding_mask.to(torch.bool)

        if self.add_bias_kv:
            if attn_mask is not None:
                attn_mask = F.pad(attn_mask, (0, 1))
            if key_padding_mask is not None:
                key_padding_mask = F.pad(key_padding_mask, (0, 1))
        if self.add_zero_attn:
            k = torch.cat([k, k.new_zeros((1,) + tuple(k.shape[1:]))], dim=0)
            v = torch.cat([v, v.new_zeros((1,) + tuple(v.shape[1:]))], dim=0)
            if attn_mask is not None:
                attn_mask = F.pad(attn_mask, (0, 1))
            if key_padding_mask is not None:
                key_padding_mask = F.pad(key_padding_mask, (0, 1))
        src_len = k.shape[0]
        if key_padding_mask is not None:
            assert key_padding_mask.shape == (bsz, src_len)

        # [N, H, L, hd]
        q = q.reshape(tgt_len, bsz, H, hd).permute(1, 2, 0, 3)
        k = k.reshape(src_len, bsz, H, hd).permute(1, 2, 0, 3)
        v = v.reshape(src_len, bsz, H, hd).permute(1, 2, 0, 3)

        # one additive mask [N or 1, H or 1, L, S] out of the two the caller may give
        mask = None
        if attn_mask is not None:
            m = attn_mask.view(1, 1, tgt_len, src_len) if attn_mask.shape[0] == 1 else attn_mask.view(bsz, H, tgt_len, src_len)
            mask = torch.zeros_like(m, dtype=q.dtype).masked_fill_(m, float("-inf")) if m.dtype == torch.bool else m.to(q.dtype)
        if key_padding_mask is not None:
            pad = torch.zeros(bsz, 1, 1, src_len, dtype=q.dtype, device=q.device)
            pad.masked_fill_(key_padding_mask.view(bsz, 1, 1, src_len), float("-inf"))
            mask = pad if mask is None else mask + pad

        if need_weights:
            scores = torch.matmul(q * (float(hd) ** -0.5), k.transpose(-2, -1))
            if mask is not None:
                scores = scores + mask
            weights = self.dropout(F.softmax(scores, dim=-1))
            attn = torch.matmul(weights, v)
        else:
            weights = None
            attn = F.scaled_dot_product_attention(
                q, k, v, attn_mask=mask, dropout_p=self.dropout.p if self.training else 0.0
            )

        attn = attn.permute(2, 0, 1, 3).reshape(tgt_len, bsz, embed_dim)  # [L, N, E]
        if self.batch_first:
            attn = attn.transpose(0, 1)
        out = self.out_proj(attn)
        if need_weights:
            return out, weights.sum(dim=1) / H
        return out, None
