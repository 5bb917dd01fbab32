"""CPU oracle for the DP-SGD hot path. TEST INFRASTRUCTURE ONLY.

A plain-PyTorch (CPU) restatement of what the reference computes on this path, one
function per reference function, each citing the file:line it follows (paths relative
to the reference tree, ``opacus/...``). It exists to check the HIP kernels and to be
timed as the CPU baseline. Nothing in the ``opacus_amd`` package imports it; only the
tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do.

What pins each function (see ``tests/test_oracle_pins.py``):
  * linear/conv/embedding/norm-layer (Group, RMS, Layer, Instance) grad samples: batch-of-one autograd (the
    reference's own microbatch method, opacus/utils/per_sample_gradients_utils.py:96-167)
    and the invariant sum_n gs[n] == autograd's .grad for a sum loss;
  * unfold2d: exact equality with torch.nn.functional.unfold
    (opacus/tests/grad_samples/conv2d_test.py:121-153);
  * unfold3d / Conv3d grad sample: batch-of-one autograd of nn.Conv3d over strides,
    dilations, groups and "same" padding; a depth-one call equals unfold2d exactly;
  * linear ghost norm: equals the Frobenius norm of the materialised grad sample in
    float64, and the closed forms for T == 1;
  * embedding ghost norm: the three input/expected triples of
    opacus/tests/grad_samples/embedding_norm_sample_test.py:25-210 and every
    intermediate of the worked example in
    opacus/grad_sample/embedding_norm_sample.py:42-101;
  * clip_and_accumulate / add_noise / scale_grad: closed forms, batch-of-one gives a sum
    of norm C (opacus/tests/privacy_engine_test.py:302-327), C -> inf and sigma = 0
    reproduce plain SGD (:220-273);
  * EmbeddingBag grad sample: batch-of-one autograd for bags without repeated indices
    (with repeats the reference's indexed "+=" writes the row once; that is restated as it
    is and checked on a hand-computed case);
  * per-layer clipping: reduces to flat clipping for one parameter, to the plain sum for
    huge bounds, and bounds every parameter's norm by its own C_k; AdaClip's count and
    bound update: hand-checked numbers; the ghost-mode adaptive update: hand-checked
    numbers, the fixed point at the target quantile, the composition identity
    sigma'^-2 + (2 n/20)^-2 == sigma^-2, and coefficients that scale every clipped sample
    to exactly the new bound;
  * tied embedding / projection norm: it is the materialised definition (sum of the two
    pinned gradients); checked against autograd's gradient of the shared table with a batch
    of one, and against |G_emb|^2 + |G_head|^2 + 2 cross from the two pinned ghost norms;
  * Philox4x32-10: the Random123 known-answer vectors.
No function here is "parity unpinned".
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F

# --------------------------------------------------------------------------------------
# Hook glue
# --------------------------------------------------------------------------------------


def scale_backprops(backprops: torch.Tensor, n: int, loss_reduction: str) -> torch.Tensor:
    """Backprops as the samplers see them: multiplied by the batch size for a mean loss.

    opacus/grad_sample/grad_sample_module.py:402-411 (a full extra pass over the tensor).
    """
    if loss_reduction == "mean":
        return backprops * n
    if loss_reduction == "sum":
        return backprops
    raise ValueError(f"loss_reduction = {loss_reduction}. Only 'sum' and 'mean' losses are supported")


def store_grad_sample(gs: torch.Tensor, max_batch_len: int) -> torch.Tensor:
    """First store of a grad sample in a backward pass: zero-filled buffer, then a copy.

    opacus/grad_sample/grad_sample_module.py:61-66.
    """
    buf = torch.zeros(torch.Size([max_batch_len]) + gs.shape[1:], device=gs.device, dtype=gs.dtype)
    buf[: gs.shape[0]] = gs
    return buf


# --------------------------------------------------------------------------------------
# nn.Linear
# --------------------------------------------------------------------------------------


def linear_grad_sample(
    activations: torch.Tensor, backprops: torch.Tensor, bias: bool = True
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """opacus/grad_sample/linear.py:41-51: weight ``einsum("n...i,n...j->nij")``, bias ``einsum("n...k->nk")``."""
    a = activations.to(backprops.dtype)  # linear.py:43
    gs_w = torch.einsum("n...i,n...j->nij", backprops, a)
    gs_b = torch.einsum("n...k->nk", backprops) if bias else None
    return gs_w, gs_b


def linear_norm_sample(
    activations: torch.Tensor, backprops: torch.Tensor, bias: bool = True
) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """opacus/grad_sample/linear.py:66-93: per-sample gradient norms without the gradients.

    2-d backprops: sqrt(|b|^2 |a|^2) and |b| (:71-79). 3-d: two T x T Gram matrices
    contracted elementwise, clamped at zero, square-rooted (:80-92). Other ranks: nothing.
    """
    a = activations.to(backprops.dtype)
    b = backprops
    if b.dim() == 2:
        g = torch.einsum("n...i,n...i->n", b, b)
        aa = torch.einsum("n...j,n...j->n", a, a)
        return torch.sqrt((g * aa).flatten()), (torch.sqrt(g.flatten()) if bias else None)
    if b.dim() == 3:
        ggT = torch.einsum("nik,njk->nij", b, b)
        aaT = torch.einsum("nik,njk->nij", a, a)
        nw = torch.sqrt(torch.einsum("n...i,n...i->n", ggT, aaT).clamp(min=0))
        nb = torch.sqrt(torch.einsum("n...i->n", ggT).clamp(min=0)) if bias else None
        return nw, nb
    return None, None


# --------------------------------------------------------------------------------------
# nn.Conv2d
# --------------------------------------------------------------------------------------


def conv2d_padding(padding, kernel_size, dilation) -> Tuple[int, int, int, int]:
    """(top, bottom, left, right) padding as unfold2d derives it.

    opacus/utils/tensor_utils.py:128-144: "same" is asymmetric with the smaller half first.
    """
    if padding == "same":
        th = dilation[0] * (kernel_size[0] - 1)
        tw = dilation[1] * (kernel_size[1] - 1)
        return th // 2, th - th // 2, tw // 2, tw - tw // 2
    if padding == "valid":
        return 0, 0, 0, 0
    return padding[0], padding[0], padding[1], padding[1]


def unfold2d(x: torch.Tensor, *, kernel_size, padding, stride, dilation) -> torch.Tensor:
    """im2col of a 4-d input: ``[n, C*kh*kw, OH*OW]``, rows ordered (c, kh, kw).

    opacus/utils/tensor_utils.py:116-172 builds it by padding and a strided view; this
    restatement gathers explicitly, index by index, so that a wrong stride or dilation
    pairing cannot hide in a shared trick.
    """
    n, C, H, W = x.shape
    kh, kw = kernel_size
    pt, pb, pl, pr = conv2d_padding(padding, kernel_size, dilation)
    oh = (H + pt + pb - (kh + (kh - 1) * (dilation[0] - 1))) // stride[0] + 1
    ow = (W + pl + pr - (kw + (kw - 1) * (dilation[1] - 1))) // stride[1] + 1
    xp = F.pad(x, (pl, pr, pt, pb))
    rows = (torch.arange(oh) * stride[0])[None, :] + (torch.arange(kh) * dilation[0])[:, None]  # [kh, oh]
    cols = (torch.arange(ow) * stride[1])[None, :] + (torch.arange(kw) * dilation[1])[:, None]  # [kw, ow]
    # out[n, c, i, j, y, x] = xp[n, c, rows[i, y], cols[j, x]]
    out = xp[:, :, rows[:, None, :, None], cols[None, :, None, :]]
    return out.reshape(n, C * kh * kw, oh * ow)


def conv2d_grad_sample(
    x: torch.Tensor,
    backprops: torch.Tensor,
    *,
    kernel_size,
    padding,
    stride,
    dilation,
    groups: int,
    bias: bool = True,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """opacus/grad_sample/conv.py:42-119, Conv2d branch.

    Unfold, contract over output positions (:102), keep the group-diagonal blocks
    (:104-112), reshape to ``[n, O, C/groups, kh, kw]``; bias sums over positions (:117).
    An empty batch returns zeros with a batch dimension of ONE (:46-53).
    """
    x = x.to(backprops.dtype)
    n, C = x.shape[0], x.shape[1]
    O = backprops.shape[1]
    kh, kw = kernel_size
    if n == 0:
        gs = torch.zeros(1, O, C // groups, kh, kw, dtype=backprops.dtype)
        return gs, (torch.zeros(1, O, dtype=backprops.dtype) if bias else None)
    U = unfold2d(x, kernel_size=kernel_size, padding=padding, stride=stride, dilation=dilation)
    b = backprops.reshape(n, -1, U.shape[-1])
    full = torch.einsum("noq,npq->nop", b, U)
    full = full.view(n, groups, -1, groups, C // groups, kh * kw)
    gs = torch.einsum("ngrg...->ngr...", full).contiguous().view(n, O, C // groups, kh, kw)
    return gs, (b.sum(dim=2) if bias else None)


def unfold3d(x: torch.Tensor, *, kernel_size, padding, stride, dilation) -> torch.Tensor:
    """im2col of a 5-d input: ``[n, C*kd*kh*kw, OD*OH*OW]``, rows ordered (c, kd, kh, kw)
    (opacus/utils/tensor_utils.py:175-279), gathered index by index. ``padding`` is a triple,
    "same" (smaller half first, :224-233) or "valid"."""
    n, C = x.shape[:2]
    pads = []
    for d in range(3):
        if padding == "same":
            total = dilation[d] * (kernel_size[d] - 1)
            pads.append((total // 2, total - total // 2))
        elif padding == "valid":
            pads.append((0, 0))
        else:
            pads.append((padding[d], padding[d]))
    xp = F.pad(x, (pads[2][0], pads[2][1], pads[1][0], pads[1][1], pads[0][0], pads[0][1]))
    idx, outs = [], []
    for d in range(3):
        size = x.shape[2 + d] + pads[d][0] + pads[d][1]
        o = (size - (dilation[d] * (kernel_size[d] - 1) + 1)) // stride[d] + 1
        outs.append(o)
        idx.append((torch.arange(o) * stride[d])[None, :] + (torch.arange(kernel_size[d]) * dilation[d])[:, None])
    zi, yi, xi = idx  # each [k, o]
    # out[n, c, a, i, j, z, y, x] = xp[n, c, zi[a, z], yi[i, y], xi[j, x]]
    out = xp[
        :, :, zi[:, None, None, :, None, None], yi[None, :, None, None, :, None], xi[None, None, :, None, None, :]
    ]
    kd, kh, kw = kernel_size
    return out.reshape(n, C * kd * kh * kw, outs[0] * outs[1] * outs[2])


def conv3d_grad_sample(
    x: torch.Tensor, backprops: torch.Tensor, *, kernel_size, padding, stride, dilation, groups: int, bias: bool = True
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """opacus/grad_sample/conv.py:89-117, Conv3d branch: unfold3d, contract over output positions,
    keep the group-diagonal blocks, reshape to ``[n, O, C/groups, kd, kh, kw]``."""
    x = x.to(backprops.dtype)
    n, C = x.shape[0], x.shape[1]
    O = backprops.shape[1]
    kd, kh, kw = kernel_size
    U = unfold3d(x, kernel_size=kernel_size, padding=padding, stride=stride, dilation=dilation)
    b = backprops.reshape(n, -1, U.shape[-1])
    full = torch.einsum("noq,npq->nop", b, U)
    full = full.view(n, groups, -1, groups, C // groups, kd * kh * kw)
    gs = torch.einsum("ngrg...->ngr...", full).contiguous().view(n, O, C // groups, kd, kh, kw)
    return gs, (b.sum(dim=2) if bias else None)


# --------------------------------------------------------------------------------------
# nn.Embedding
# --------------------------------------------------------------------------------------


def embedding_grad_sample(ids: torch.Tensor, backprops: torch.Tensor, num_embeddings: int) -> torch.Tensor:
    """opacus/grad_sample/embedding.py:40-63: scatter-add of backprop rows into ``[n, V, D]``.

    ``padding_idx`` plays no role; an empty batch gives zeros of batch dimension one (:44-46).
    """
    D = backprops.shape[-1]
    n = ids.shape[0]
    if n == 0:
        return torch.zeros(1, num_embeddings, D, dtype=backprops.dtype)
    index = ids.unsqueeze(-1).expand(*ids.shape, D).reshape(n, -1, D)
    gs = torch.zeros(n, num_embeddings, D, dtype=backprops.dtype)
    gs.scatter_add_(1, index, backprops.reshape(n, -1, D))
    return gs


def embedding_bag_grad_sample(
    index: torch.Tensor, offsets: torch.Tensor, backprops: torch.Tensor, num_embeddings: int, mode: str
) -> torch.Tensor:
    """opacus/grad_sample/embedding.py:67-94, loop and all: bag ``i`` is
    ``index[offsets[i]:offsets[i+1]]`` (the last one runs to the end); its rows receive
    ``backprops[i]`` (``/ len`` for "mean") through an indexed ``+=``, which writes a row once
    even when the index repeats."""
    nbags = offsets.shape[0]
    gs = torch.zeros(nbags, num_embeddings, backprops.shape[-1], dtype=backprops.dtype)
    for i in range(nbags):
        begin = int(offsets[i])
        end = int(offsets[i + 1]) if i < nbags - 1 else index.shape[0]
        if mode == "sum":
            gs[i][index[begin:end]] += backprops[i]
        elif mode == "mean":
            gs[i][index[begin:end]] += backprops[i] / (end - begin)
    return gs


def embedding_unique_pairs(ids: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """opacus/grad_sample/embedding_norm_sample.py:107-129, the integer stage.

    Pairs every id with its row (sample) index and returns the sorted unique pairs
    ``[U, 2]`` and, for every position, the index of its pair in that list.
    """
    ids2 = ids.reshape(ids.shape[0], -1)
    nrows, ncols = ids2.shape
    row = torch.repeat_interleave(torch.arange(nrows), ncols).unsqueeze(-1)
    paired = torch.cat([row, ids2.reshape(-1, 1)], dim=1)
    if paired.shape[0] == 0:
        return paired, torch.zeros(0, dtype=torch.int64)
    uniq, inverse = torch.unique(paired, dim=0, return_inverse=True, sorted=True)
    return uniq, inverse


def tied_embedding_norm_sample(
    ids: torch.Tensor,
    emb_backprops: torch.Tensor,
    head_activations: torch.Tensor,
    head_backprops: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """A table shared by nn.Embedding and nn.Linear, by the materialising path's rule that the
    uses of a parameter add up (opacus/grad_sample/grad_sample_module.py:58-59): forms both
    per-sample gradients ``[n, V, D]`` (embedding.py:40-63, linear.py:41-51), and returns the
    norm of their sum and the inner product of the two, per sample. This is the brute-force
    definition; the reference itself raises for tied parameters under ghost clipping
    (grad_sample_module_fast_gradient_clipping.py:172-179)."""
    V = head_backprops.shape[-1]
    g_emb = embedding_grad_sample(ids, emb_backprops, V)
    g_head, _ = linear_grad_sample(head_activations, head_backprops, bias=False)
    norm = (g_emb + g_head).flatten(1).norm(dim=1)
    cross = (g_emb * g_head).flatten(1).sum(dim=1)
    return norm, cross


def embedding_norm_sample(ids: torch.Tensor, backprops: torch.Tensor) -> Dict[str, torch.Tensor]:
    """opacus/grad_sample/embedding_norm_sample.py:103-151.

    Sums backprop rows that share (sample, id), squares, sums per sample, square root.
    Returns the final norms and the intermediates the reference's docstring lists.
    """
    nrows = ids.shape[0]
    g = backprops.reshape(-1, backprops.size(-1))
    uniq, inverse = embedding_unique_pairs(ids)
    summed = torch.zeros(uniq.size(0), g.size(-1), dtype=g.dtype).index_add(0, inverse, g)
    sq = torch.sum(summed**2, dim=1)
    result = torch.zeros(nrows, dtype=g.dtype)
    result.scatter_add_(0, uniq[:, 0], sq)
    return {
        "unique_paired_indices": uniq,
        "new_index_positions": inverse,
        "summed_gradients": summed,
        "sqr_gradient_sum": sq,
        "result": result,
        "result_sqrt": torch.sqrt(result),
    }


# --------------------------------------------------------------------------------------
# Normalisation layers
# --------------------------------------------------------------------------------------


def group_norm_grad_sample(
    x: torch.Tensor, backprops: torch.Tensor, num_groups: int, eps: float
) -> Tuple[torch.Tensor, torch.Tensor]:
    """opacus/grad_sample/group_norm.py:41-46: ``sum_spatial group_norm(x) * b`` and ``sum_spatial b``."""
    gs_w = torch.einsum("ni...->ni", F.group_norm(x, num_groups, eps=eps) * backprops)
    gs_b = torch.einsum("ni...->ni", backprops)
    return gs_w, gs_b


def layer_norm_grad_sample(
    x: torch.Tensor, backprops: torch.Tensor, normalized_shape: Sequence[int], eps: float
) -> Tuple[torch.Tensor, torch.Tensor]:
    """opacus/grad_sample/layer_norm.py:41-50: ``layer_norm(x) * b`` and ``b`` summed over all but
    the batch and the normalised dimensions."""
    k = len(normalized_shape)
    prod = F.layer_norm(x, tuple(normalized_shape), eps=eps) * backprops
    if prod.dim() == k + 1:
        return prod, backprops
    dims = list(range(1, prod.dim() - k))
    return prod.sum(dim=dims), backprops.sum(dim=dims)


def instance_norm_grad_sample(x: torch.Tensor, backprops: torch.Tensor, eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """opacus/grad_sample/instance_norm.py:50-55: ``instance_norm(x) * b`` and ``b`` summed over
    the spatial dimensions."""
    return torch.einsum("ni...->ni", F.instance_norm(x, eps=eps) * backprops), torch.einsum("ni...->ni", backprops)


def rms_norm_grad_sample(
    x: torch.Tensor, backprops: torch.Tensor, normalized_shape: Sequence[int], eps: Optional[float]
) -> torch.Tensor:
    """opacus/grad_sample/rms_norm.py:42-47: ``rms_norm(x) * b`` summed over all but batch and feature dims."""
    prod = F.rms_norm(x, tuple(normalized_shape), eps=eps) * backprops
    k = len(normalized_shape)
    if prod.dim() == k + 1:
        return prod
    # opacus/utils/tensor_utils.py:87-113 (sum_over_all_but_batch_and_last_n)
    return prod.sum(dim=list(range(1, prod.dim() - k)))


# --------------------------------------------------------------------------------------
# Ghost clipping
# --------------------------------------------------------------------------------------


def per_sample_norm(norm_samples: Sequence[torch.Tensor]) -> torch.Tensor:
    """opacus/grad_sample/grad_sample_module_fast_gradient_clipping.py:142-150: 2-norm over the stack."""
    return torch.stack(list(norm_samples), dim=0).norm(2, dim=0)


def clipping_coef(norm_samples: Sequence[torch.Tensor], max_grad_norm: float) -> torch.Tensor:
    """opacus/grad_sample/grad_sample_module_fast_gradient_clipping.py:137-140."""
    return (max_grad_norm / (per_sample_norm(norm_samples) + 1e-6)).clamp(max=1.0)


# --------------------------------------------------------------------------------------
# DPOptimizer
# --------------------------------------------------------------------------------------


def clip_and_accumulate(
    grad_samples: Sequence[torch.Tensor],
    max_grad_norm: float,
    param_dtypes: Optional[Sequence[torch.dtype]] = None,
    summed: Optional[Sequence[Optional[torch.Tensor]]] = None,
) -> Tuple[torch.Tensor, torch.Tensor, List[torch.Tensor]]:
    """opacus/optimizers/optimizer.py:432-475.

    Per-parameter per-sample norms (:444-446), their 2-norm over parameters (:452), the
    clip factor ``min(1, C / (norm + 1e-6))`` (:453-455), the clip-weighted sum over the
    batch in the parameter's dtype (:464-468), added to a previous ``summed_grad`` if there
    is one (:470-473). Returns (per-sample norms, clip factors, summed grads).
    """
    if len(grad_samples[0]) == 0:
        norms = torch.zeros((0,))
        clip = torch.zeros((0,))
    else:
        per_param = [g.reshape(len(g), -1).norm(2, dim=-1) for g in grad_samples]
        norms = torch.stack(per_param, dim=1).norm(2, dim=1)
        clip = (max_grad_norm / (norms + 1e-6)).clamp(max=1.0)
    out = []
    for k, g in enumerate(grad_samples):
        dt = param_dtypes[k] if param_dtypes is not None else g.dtype
        grad = torch.einsum("i,i...", clip.to(dt), g.to(dt))
        if summed is not None and summed[k] is not None:
            grad = summed[k] + grad
        out.append(grad)
    return norms, clip, out


def per_layer_clip_and_accumulate(
    grad_samples: Sequence[torch.Tensor], max_grad_norms: Sequence[float]
) -> Tuple[List[torch.Tensor], List[torch.Tensor]]:
    """opacus/optimizers/perlayeroptimizer.py:58-76: every parameter clipped on its own norm with
    its own bound. Returns (clip factors per parameter, summed grads)."""
    clips, out = [], []
    for g, c in zip(grad_samples, max_grad_norms):
        norms = g.reshape(len(g), -1).norm(2, dim=-1)
        clip = (c / (norms + 1e-6)).clamp(max=1.0)
        clips.append(clip)
        out.append(torch.einsum("i,i...", clip, g))
    return clips, out


def adaclip_update(
    clip: torch.Tensor, max_grad_norm: float, target_quantile: float, learning_rate: float, min_bound: float,
    max_bound: float, count_noise: float = 0.0,
) -> Tuple[float, float]:
    """opacus/optimizers/adaclipoptimizer.py:119-121, 181-194: the unclipped count
    ``n - #(clip < 1)`` (plus its noise) and the bound after one geometric update, kept inside
    ``[min_bound, max_bound]``. Returns (noisy count, new bound)."""
    n = len(clip)
    count = float(n - int((clip < 1).sum())) + count_noise
    new = max_grad_norm * math.exp(-learning_rate * (count / n - target_quantile))
    return count, min(max(new, min_bound), max_bound)


def ghost_adaptive_update(
    per_sample_norms: torch.Tensor,
    max_grad_norm: float,
    target_quantile: float,
    learning_rate: float,
    min_bound: float,
    max_bound: float,
    noise_multiplier: float,
    count_noise: float = 0.0,
) -> Tuple[float, float, torch.Tensor]:
    """opacus/utils/adaptive_clipping/adaptive_clipping_utils.py:77-175: the ghost-clipping
    variant of adaptive clipping. Counts ``norm <= C`` (plus ``count_noise``, a draw of
    N(0, (n/20)^2)), moves C geometrically, raises the noise multiplier to
    ``(sigma^-2 - (2 n/20)^-2)^-1/2``, and returns the coefficients of the second backward
    pass from the *new* bound: 1 where ``norm <= C'``, else ``C' / norm`` (no 1e-6 here).
    Returns (new bound, new noise multiplier, coefficients)."""
    n = len(per_sample_norms)
    count = float((per_sample_norms <= max_grad_norm).sum()) + count_noise
    new = max_grad_norm * math.exp(-learning_rate * (count / n - target_quantile))
    new = min(max(new, min_bound), max_bound)
    std = n / 20.0
    sigma = noise_multiplier
    if noise_multiplier > 0:
        sigma = (noise_multiplier ** (-2) - (2.0 * std) ** (-2)) ** (-0.5)
    coeff = torch.where(per_sample_norms <= new, torch.ones_like(per_sample_norms), new / per_sample_norms)
    return new, sigma, coeff


def generate_noise(std: float, reference: torch.Tensor, generator=None, secure_mode: bool = False) -> torch.Tensor:
    """opacus/optimizers/optimizer.py:138-169: zeros for std == 0, else one normal draw
    (or, in secure mode, one discarded draw then four summed and halved)."""
    zeros = torch.zeros(reference.shape, dtype=reference.dtype)
    if std == 0:
        return zeros
    if secure_mode:
        torch.normal(mean=0, std=std, size=(1, 1), generator=generator)
        total = zeros
        for _ in range(4):
            total += torch.normal(mean=0, std=std, size=reference.shape, generator=generator)
        return total / 2
    return torch.normal(mean=0, std=std, size=reference.shape, generator=generator, dtype=reference.dtype)


def add_noise_and_scale(
    summed: Sequence[torch.Tensor],
    shapes: Sequence[torch.Size],
    noise_multiplier: float,
    max_grad_norm: float,
    expected_batch_size: int,
    loss_reduction: str = "mean",
    accumulated_iterations: int = 1,
    generator=None,
    secure_mode: bool = False,
) -> List[torch.Tensor]:
    """opacus/optimizers/optimizer.py:477-504: ``grad = (summed + noise).view_as(p)``, then for a
    mean loss ``grad /= expected_batch_size * accumulated_iterations``."""
    grads = []
    for s, shape in zip(summed, shapes):
        noise = generate_noise(noise_multiplier * max_grad_norm, s, generator, secure_mode)
        g = (s + noise).view(shape)
        if loss_reduction == "mean":
            g = g / (expected_batch_size * accumulated_iterations)
        grads.append(g)
    return grads


# --------------------------------------------------------------------------------------
# Brute force: the reference's own microbatch method
# --------------------------------------------------------------------------------------


def microbatch_grad_sample(
    module: nn.Module, x: torch.Tensor, loss_reduction: str = "sum", batch_first: bool = True
) -> Dict[str, torch.Tensor]:
    """Per-sample gradients by running the module on one sample at a time.

    opacus/utils/per_sample_gradients_utils.py:53-93, 96-167: L1 loss against zeros, one
    backward per sample, gradients stacked; for a mean loss each microbatch gradient is
    what the sample contributes to the batch mean times the batch size, i.e. unchanged.
    """
    bdim = 0 if batch_first else 1
    n = x.shape[bdim]
    names = [k for k, p in module.named_parameters() if p.requires_grad]
    out = {k: [] for k in names}
    for i in range(n):
        xi = x.narrow(bdim, i, 1)
        module.zero_grad()
        y = module(xi)
        crit = nn.L1Loss(reduction=loss_reduction)
        loss = crit(y, torch.zeros_like(y))
        loss.backward()
        for k, p in module.named_parameters():
            if p.requires_grad:
                out[k].append(p.grad.detach().clone())
    module.zero_grad()
    return {k: torch.stack(v, dim=0) for k, v in out.items()}


# --------------------------------------------------------------------------------------
# Philox4x32-10 (the generator the HIP noise kernel uses; not part of the reference, which
# calls torch.normal: noise parity with the reference is statistical by construction)
# --------------------------------------------------------------------------------------

_M0, _M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
_W0, _W1 = np.uint32(0x9E3779B9), np.uint32(0xBB67AE85)


def philox4x32_10(counter: np.ndarray, key: np.ndarray) -> np.ndarray:
    """Philox4x32 with 10 rounds (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as
    easy as 1, 2, 3", SC'11). ``counter``: ``[..., 4]`` uint32, ``key``: ``[..., 2]`` uint32."""
    c = np.array(counter, dtype=np.uint32, copy=True)
    k = np.array(np.broadcast_to(np.asarray(key, dtype=np.uint32), c.shape[:-1] + (2,)), copy=True)
    with np.errstate(over="ignore"):
        for _ in range(10):
            p0 = _M0 * c[..., 0].astype(np.uint64)
            p1 = _M1 * c[..., 2].astype(np.uint64)
            hi0, lo0 = (p0 >> np.uint64(32)).astype(np.uint32), p0.astype(np.uint32)
            hi1, lo1 = (p1 >> np.uint64(32)).astype(np.uint32), p1.astype(np.uint32)
            c = np.stack([hi1 ^ c[..., 1] ^ k[..., 0], lo1, hi0 ^ c[..., 3] ^ k[..., 1], lo0], axis=-1)
            k = np.stack([k[..., 0] + _W0, k[..., 1] + _W1], axis=-1)
    return c


def philox_normal(P: int, seed: int, offset: int) -> np.ndarray:
    """The N(0,1) stream of the HIP noise kernel for elements 0..P-1 (float32).

    Group g = elements 4g..4g+3; counter = (g lo, g hi, offset lo, offset hi); key = seed;
    the four outputs (x, y, z, w) give Box-Muller pairs (x, y) -> elements 0, 1 and
    (z, w) -> elements 2, 3 with u = bits * 2^-32 + 2^-33.
    """
    ng = (P + 3) // 4
    g = np.arange(ng, dtype=np.uint64)
    ctr = np.stack(
        [
            (g & np.uint64(0xFFFFFFFF)).astype(np.uint32),
            (g >> np.uint64(32)).astype(np.uint32),
            np.full(ng, offset & 0xFFFFFFFF, dtype=np.uint32),
            np.full(ng, (offset >> 32) & 0xFFFFFFFF, dtype=np.uint32),
        ],
        axis=-1,
    )
    key = np.array([seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF], dtype=np.uint32)
    r = philox4x32_10(ctr, key)
    u = r.astype(np.float32) * np.float32(2.3283064365386963e-10) + np.float32(1.1641532182693481e-10)
    r0 = np.sqrt(np.float32(-2.0) * np.log(u[:, 0]))
    r1 = np.sqrt(np.float32(-2.0) * np.log(u[:, 2]))
    t0 = np.float32(6.2831853071795865) * u[:, 1]
    t1 = np.float32(6.2831853071795865) * u[:, 3]
    z = np.stack([r0 * np.cos(t0), r0 * np.sin(t0), r1 * np.cos(t1), r1 * np.sin(t1)], axis=-1)
    return z.reshape(-1)[:P].astype(np.float32)
