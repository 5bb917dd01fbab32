"""Tensor-level wrappers over the C ABI of ``libdpsgd_hip.so``.

Each function checks devices, dtypes and shapes, makes inputs dense, allocates the
outputs (and the workspace the entry point asks for) with torch, and enqueues the
HIP kernels on torch's current stream of the tensors' device. Tensors must live on
the GPU: there is no CPU implementation behind these calls.
"""

from __future__ import annotations

import ctypes
import math
from contextlib import contextmanager
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import DPK_BF16, DPK_F32, DPK_MULTI_MAX, check, lib

_DTYPES = {torch.float32: DPK_F32, torch.bfloat16: DPK_BF16}


def supported_dtype(dtype: torch.dtype) -> bool:
    """float32 and bfloat16 have kernels of their own; float16 tensors are widened to float32 on
    the way in (exact) and results narrowed on the way out (:func:`widen`, the optimizer wrappers
    below, ``grad_sample_module.call_sampler``)."""
    return dtype in _DTYPES or dtype is torch.float16


def native_dtype(dtype: torch.dtype) -> bool:
    """Whether the kernels read and write the dtype directly (float32, bfloat16)."""
    return dtype in _DTYPES


def widen(t):
    """float16 -> float32 (every float16 value is a float32 value); anything else as it is."""
    return t.float() if isinstance(t, torch.Tensor) and t.dtype is torch.float16 else t


def _any_half(*lists) -> bool:
    return any(t is not None and t.dtype is torch.float16 for ts in lists for t in ts)


def _narrow_back(targets, wide) -> None:
    for t, w in zip(targets, wide):
        if t is not w:
            t.copy_(w)


def _code(t_or_dtype) -> int:
    dt = t_or_dtype.dtype if isinstance(t_or_dtype, torch.Tensor) else t_or_dtype
    try:
        return _DTYPES[dt]
    except KeyError:
        raise TypeError(f"dpk kernels take float32 or bfloat16 tensors (float16 through kernels.widen), got {dt}") from None


def _need_gpu(*tensors: torch.Tensor) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "opacus_amd runs on the GPU only (HIP kernels, no CPU fallback); got a tensor on "
                f"{t.device}"
            )
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
    return dev


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(dev: torch.device):
    """torch's current stream on ``dev`` as a raw handle (the direct binding where torch has it:
    building a ``torch.cuda.Stream`` object per kernel launch is a visible cost for small models)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(dev.index if dev.index is not None else torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def _ws(nbytes: int, dev: torch.device) -> Tuple[Optional[torch.Tensor], int]:
    if nbytes == 0:
        return None, 0
    t = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    return t, nbytes


# ---- optional per-kernel timing (HIP events on the launch stream) -------------------
_TIMING: Optional[Dict[str, List[Tuple[torch.cuda.Event, torch.cuda.Event]]]] = None
_TIMING_ONLY: Optional[frozenset] = None


@contextmanager
def record_kernel_times(only=None):
    """Collects (start, end) event pairs around every wrapper call made inside the block, or
    around the calls of the wrappers named in ``only`` (two event records per call are not
    free for a launch-bound model).

    Yields a dict ``name -> [(start, end), ...]``; after a device synchronize,
    ``start.elapsed_time(end)`` is the duration in ms of that call's kernels.
    """
    global _TIMING, _TIMING_ONLY
    prev, _TIMING = _TIMING, {}
    prev_only, _TIMING_ONLY = _TIMING_ONLY, (None if only is None else frozenset(only))
    try:
        yield _TIMING
    finally:
        _TIMING, _TIMING_ONLY = prev, prev_only


@contextmanager
def _timed(name: str, dev: torch.device):
    if _TIMING is None or (_TIMING_ONLY is not None and name not in _TIMING_ONLY):
        yield
        return
    with torch.cuda.device(dev):
        s = torch.cuda.Event(enable_timing=True)
        e = torch.cuda.Event(enable_timing=True)
        s.record()
        yield
        e.record()
    _TIMING.setdefault(name, []).append((s, e))


def _dense(t: torch.Tensor) -> torch.Tensor:
    return t if t.is_contiguous() else t.contiguous()


# ---- nn.Linear ----------------------------------------------------------------------
def linear_grad_sample(
    backprops: torch.Tensor,
    activations: torch.Tensor,
    scale: float = 1.0,
    want_sumsq: bool = True,
    out_dtype: Optional[torch.dtype] = None,
    tile: int = _lib.DPK_TILE_AUTO,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """``gs[n,i,j] = scale * sum_t b[n,t,i] a[n,t,j]`` and ``sum_ij gs[n]^2``.

    ``backprops`` is ``[n, *, out]``, ``activations`` ``[n, *, in]`` with the same middle dims.
    ``tile`` (128 or 256) names the block tile of the bf16 contraction kernel instead of
    leaving the choice to the library; tests use it.
    """
    dev = _need_gpu(backprops, activations)
    if activations.dtype != backprops.dtype:
        activations = activations.to(backprops.dtype)
    n, out_f, in_f = backprops.shape[0], backprops.shape[-1], activations.shape[-1]
    b = _dense(backprops).reshape(n, -1, out_f) if n else backprops.reshape(0, 1, out_f)
    a = _dense(activations).reshape(n, -1, in_f) if n else activations.reshape(0, 1, in_f)
    T = b.shape[1]
    if a.shape[1] != T:
        raise ValueError(f"activations {tuple(activations.shape)} and backprops {tuple(backprops.shape)} disagree")
    out_dtype = out_dtype or backprops.dtype
    gs = torch.empty((n, out_f, in_f), dtype=out_dtype, device=dev)
    sumsq = torch.empty((n,), dtype=torch.float32, device=dev) if want_sumsq else None
    if n == 0:
        return gs, sumsq
    L = lib()
    ws, wsb = _ws(L.dpk_linear_gs_workspace_bytes(n, T, out_f, in_f) if want_sumsq else 0, dev)
    with _timed("linear_gs", dev):
        check(
            "dpk_linear_gs",
            L.dpk_linear_gs(
                _ptr(b), _ptr(a), _code(b), _ptr(gs), _code(gs), _ptr(sumsq), n, T, out_f, in_f,
                float(scale), int(tile), _ptr(ws), wsb, _stream(dev),
            ),
        )
    return gs, sumsq


def linear_weighted_sum_takes(backprops: torch.Tensor, activations: torch.Tensor) -> bool:
    """Whether the pair goes to the bf16 contraction with the coefficients on its accumulators
    (and may be pooled by :func:`linear_weighted_sum_multi`): bf16 on the GPU, whole k tiles of 32
    positions per sample, feature counts that are multiples of 8 above 64. Any other pair
    :func:`linear_weighted_sum` sends to the fp32 MFMA kernel with weighted rows."""
    if not (backprops.is_cuda and backprops.dtype == torch.bfloat16 and activations.dtype == torch.bfloat16):
        return False
    if backprops.dim() < 3 or backprops.shape[0] == 0 or backprops.shape[:-1] != activations.shape[:-1]:
        return False
    n, out_f, in_f = backprops.shape[0], backprops.shape[-1], activations.shape[-1]
    T = backprops.numel() // (n * out_f)
    return T % 32 == 0 and T >= 32 and out_f % 8 == 0 and in_f % 8 == 0 and out_f > 64 and in_f > 64


def linear_weighted_sum(
    backprops: torch.Tensor,
    activations: torch.Tensor,
    coef: torch.Tensor,
    scale: float = 1.0,
    pieces: Optional[int] = None,
    out_dtype: Optional[torch.dtype] = None,
) -> torch.Tensor:
    """``sum_n coef[n] * scale * b[n]^T a[n]`` as ``[out, in]``: the clip-weighted sum of a Linear
    layer's per-sample gradients in one contraction over samples and positions, for fp32 and
    bf16 operands of any shape (see :func:`linear_weighted_sum_takes` for the two kernels behind
    it). ``pieces`` cuts the samples (or rows) into that many runs whose fp32 sums a second kernel
    adds (default: 4 for a layer with at most 256 output tiles of 128 x 128, which alone would not
    fill the GPU twice over, when n allows; else 1)."""
    dev = _need_gpu(backprops, activations, coef)
    if activations.dtype != backprops.dtype:
        activations = activations.to(backprops.dtype)
    if not native_dtype(backprops.dtype):
        raise TypeError(f"linear_weighted_sum takes float32 and bfloat16, not {backprops.dtype}")
    n, out_f, in_f = backprops.shape[0], backprops.shape[-1], activations.shape[-1]
    b = _dense(backprops).reshape(n, -1, out_f)
    a = _dense(activations).reshape(n, -1, in_f)
    T = b.shape[1]
    if a.shape[1] != T:
        raise ValueError(f"activations {tuple(activations.shape)} and backprops {tuple(backprops.shape)} disagree")
    c = _dense(coef.to(torch.float32)).reshape(-1)
    if c.numel() != n:
        raise ValueError(f"{c.numel()} coefficients for {n} samples")
    if pieces is None:
        few_tiles = -(-out_f // 128) * -(-in_f // 128) <= 256
        # the kernels with the coefficients on the accumulators cut along whole samples, the one with
        # weighted rows anywhere
        per_sample = linear_weighted_sum_takes(b, a) or (
            b.dtype == torch.float32 and T % 16 == 0 and out_f % 4 == 0 and in_f % 8 == 0 and out_f > 64 and in_f > 64
        )
        pieces = 4 if few_tiles and (out_f * in_f) % 4 == 0 and (n % 4 == 0 or not per_sample) and n * T >= 256 else 1
    out = torch.empty((out_f, in_f), dtype=out_dtype or backprops.dtype, device=dev)
    L = lib()
    ws, wsb = _ws(L.dpk_linear_weighted_sum_workspace_bytes(n, T, out_f, in_f, _code(b), int(pieces)), dev)
    with _timed("linear_weighted_sum", dev):
        check(
            "dpk_linear_weighted_sum",
            L.dpk_linear_weighted_sum(
                _ptr(b), _ptr(a), _code(b), _ptr(c), _ptr(out), _code(out), n, T, out_f, in_f, float(scale),
                int(pieces), _ptr(ws), wsb, _stream(dev),
            ),
        )
    return out


def linear_weighted_sum_multi(
    items: Sequence[Tuple[torch.Tensor, torch.Tensor, torch.Tensor, float]],
    out_dtype: Optional[torch.dtype] = None,
    pooled: Optional[bool] = None,
) -> List[torch.Tensor]:
    """:func:`linear_weighted_sum` for several layers in one call: each item is ``(backprops,
    activations, coef, scale)`` (every pair one that :func:`linear_weighted_sum_takes`); returns
    the ``[out, in]`` sums in order. The block tiles of all layers are one pool of work, so the
    GPU stays full across layers whose own tile count does not fill it in whole rounds; a small
    pool (a two-layer MLP) has its samples cut into pieces inside the call
    (``pooled=False`` calls layer by layer instead)."""
    if not items:
        return []
    dev = _need_gpu(*[t for it in items for t in it[:3]])
    out_dtype = out_dtype or items[0][0].dtype
    if pooled is None:
        pooled = True
    if not pooled:
        return [linear_weighted_sum(b, a, c, scale=scale, out_dtype=out_dtype) for b, a, c, scale in items]
    table = (_lib.WsumLayer * len(items))()
    keep, outs = [], []
    for row, (bp, act, coef, scale) in zip(table, items):
        n, out_f, in_f = bp.shape[0], bp.shape[-1], act.shape[-1]
        b = _dense(bp).reshape(n, -1, out_f)
        a = _dense(act).reshape(n, -1, in_f)
        if a.shape[1] != b.shape[1] or b.dtype != torch.bfloat16 or a.dtype != torch.bfloat16:
            raise ValueError(f"activations {tuple(act.shape)} {act.dtype} and backprops {tuple(bp.shape)} {bp.dtype} disagree or are not bfloat16")
        c = _dense(coef.to(torch.float32)).reshape(-1)
        if c.numel() != n:
            raise ValueError(f"{c.numel()} coefficients for {n} samples")
        out = torch.empty((out_f, in_f), dtype=out_dtype, device=dev)
        keep.append((b, a, c))
        outs.append(out)
        row.b, row.a, row.coef, row.out_sum = b.data_ptr(), a.data_ptr(), c.data_ptr(), out.data_ptr()
        row.n, row.T, row.out, row.inp, row.scale = n, b.shape[1], out_f, in_f, float(scale)
    L = lib()
    ws, wsb = _ws(L.dpk_linear_weighted_sum_multi_workspace_bytes(table, len(items)), dev)
    with _timed("linear_weighted_sum", dev):
        check(
            "dpk_linear_weighted_sum_multi",
            L.dpk_linear_weighted_sum_multi(table, len(items), DPK_BF16, _code(out_dtype), _ptr(ws), wsb, _stream(dev)),
        )
    del keep
    return outs


def linear_bias_weighted_sum(
    backprops: torch.Tensor, coef: torch.Tensor, scale: float = 1.0, out_dtype: Optional[torch.dtype] = None
) -> torch.Tensor:
    """``scale * sum_n coef[n] * sum_t b[n, t, :]`` as ``[out]``: the clip-weighted sum of a Linear
    layer's per-sample bias gradients, one pass over the backprops."""
    dev = _need_gpu(backprops, coef)
    if not native_dtype(backprops.dtype):
        raise TypeError(f"linear_bias_weighted_sum takes float32 and bfloat16, not {backprops.dtype}")
    n, out_f = backprops.shape[0], backprops.shape[-1]
    b = _dense(backprops).reshape(n, -1, out_f)
    T = b.shape[1]
    c = _dense(coef.to(torch.float32)).reshape(-1)
    if c.numel() != n:
        raise ValueError(f"{c.numel()} coefficients for {n} samples")
    out = torch.empty((out_f,), dtype=out_dtype or backprops.dtype, device=dev)
    L = lib()
    ws, wsb = _ws(L.dpk_linear_bias_weighted_sum_workspace_bytes(n, T, out_f), dev)
    with _timed("linear_bias_weighted_sum", dev):
        check(
            "dpk_linear_bias_weighted_sum",
            L.dpk_linear_bias_weighted_sum(
                _ptr(b), _code(b), _ptr(c), _ptr(out), _code(out), n, T, out_f, float(scale), _ptr(ws), wsb, _stream(dev)
            ),
        )
    return out


def _with_sumsq(gs: torch.Tensor, sumsq: torch.Tensor) -> torch.Tensor:
    """Leaves the per-sample sum of squares on the tensor it describes, with the tensor's
    version, so that the optimizer's norm pass can use it while nobody has written to ``gs``."""
    gs._dpk_sumsq = sumsq
    gs._dpk_sumsq_version = gs._version
    return gs


def linear_bias_grad_sample(
    backprops: torch.Tensor, scale: float = 1.0, out_dtype: Optional[torch.dtype] = None
) -> torch.Tensor:
    """``gs[n,k] = scale * sum over middle dims of b[n,*,k]``; its per-sample sum of squares
    rides on the result for the optimizer."""
    dev = _need_gpu(backprops)
    n, out_f = backprops.shape[0], backprops.shape[-1]
    gs = torch.empty((n, out_f), dtype=out_dtype or backprops.dtype, device=dev)
    if n == 0:
        return gs
    sumsq = torch.empty((n,), dtype=torch.float32, device=dev)
    b = _dense(backprops).reshape(n, -1, out_f)
    with _timed("linear_bias_gs", dev):
        check(
            "dpk_linear_bias_gs",
            lib().dpk_linear_bias_gs(
                _ptr(b), _code(b), _ptr(gs), _code(gs), _ptr(sumsq), n, b.shape[1], out_f, float(scale), _stream(dev)
            ),
        )
    return _with_sumsq(gs, sumsq)


def linear_ghost_norm(
    backprops: torch.Tensor,
    activations: torch.Tensor,
    scale: float = 1.0,
    want_weight: bool = True,
    want_bias: bool = False,
    route: int = _lib.DPK_ROUTE_AUTO,
) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Per-sample norms (fp32) of the Linear weight and bias gradients without forming them.
    ``route`` (``DPK_ROUTE_GRAM`` / ``DPK_ROUTE_DIRECT``) names the kernel family instead of
    leaving the choice to the library; tests use it."""
    dev = _need_gpu(backprops, activations)
    if activations.dtype != backprops.dtype:
        activations = activations.to(backprops.dtype)
    n, out_f, in_f = backprops.shape[0], backprops.shape[-1], activations.shape[-1]
    nw = torch.empty((n,), dtype=torch.float32, device=dev) if want_weight else None
    nb = torch.empty((n,), dtype=torch.float32, device=dev) if want_bias else None
    if n == 0 or not (want_weight or want_bias):
        return nw, nb
    b = _dense(backprops).reshape(n, -1, out_f)
    a = _dense(activations).reshape(n, -1, in_f)
    T = b.shape[1]
    if a.shape[1] != T:
        raise ValueError(f"activations {tuple(activations.shape)} and backprops {tuple(backprops.shape)} disagree")
    L = lib()
    ws, wsb = _ws(L.dpk_linear_ghost_norm_workspace_bytes(n, T, out_f, in_f), dev)
    with _timed("linear_ghost_norm", dev):
        check(
            "dpk_linear_ghost_norm",
            L.dpk_linear_ghost_norm(
                _ptr(b), _ptr(a), _code(b), _ptr(nw), _ptr(nb), n, T, out_f, in_f, float(scale),
                int(route), _ptr(ws), wsb, _stream(dev),
            ),
        )
    return nw, nb


def linear_ghost_norm_multi(
    items: Sequence[Tuple[torch.Tensor, torch.Tensor, float, Optional[torch.Tensor], Optional[torch.Tensor]]],
) -> None:
    """Ghost norms of several Linear layers in one call. Each item is ``(backprops, activations,
    scale, norm_w, norm_b)`` with ``norm_w`` / ``norm_b`` preallocated float32 ``[n]`` tensors (or
    None) that receive the results. All items share the batch size, dtype and device; the tile
    pairs of all layers fill the device together instead of layer by layer."""
    items = [it for it in items if it[3] is not None or it[4] is not None]
    if not items:
        return
    dev = _need_gpu(*[t for it in items for t in (it[0], it[1])])
    n, dt = items[0][0].shape[0], items[0][0].dtype
    L = lib()
    for lo in range(0, len(items), _lib.DPK_GHOST_MULTI_MAX):
        chunk = items[lo : lo + _lib.DPK_GHOST_MULTI_MAX]
        table = (_lib.GhostLayer * len(chunk))()
        keep = []
        for row, (bp, act, scale, nw, nb) in zip(table, chunk):
            if bp.shape[0] != n or bp.dtype != dt:
                raise ValueError("layers of one linear_ghost_norm_multi call must share batch size and dtype")
            if act.dtype != dt:
                act = act.to(dt)
            out_f, in_f = bp.shape[-1], act.shape[-1]
            b = _dense(bp).reshape(n, -1, out_f)
            a = _dense(act).reshape(n, -1, in_f)
            if a.shape[1] != b.shape[1]:
                raise ValueError(f"activations {tuple(act.shape)} and backprops {tuple(bp.shape)} disagree")
            for o in (nw, nb):
                if o is not None and (o.dtype != torch.float32 or o.numel() != n or not o.is_contiguous()):
                    raise ValueError("norm outputs must be dense float32 [n] tensors")
            keep.append((a, b))
            row.b, row.a = b.data_ptr(), a.data_ptr()
            row.norm_w = None if nw is None else nw.data_ptr()
            row.norm_b = None if nb is None else nb.data_ptr()
            row.T, row.out, row.inp, row.scale = b.shape[1], out_f, in_f, float(scale)
        if n == 0:
            continue
        ws, wsb = _ws(L.dpk_linear_ghost_norm_multi_workspace_bytes(table, len(chunk), n), dev)
        with _timed("linear_ghost_norm", dev):
            check(
                "dpk_linear_ghost_norm_multi",
                L.dpk_linear_ghost_norm_multi(table, len(chunk), _code(dt), n, _ptr(ws), wsb, _stream(dev)),
            )
        del keep


# ---- nn.Conv2d ----------------------------------------------------------------------
def conv2d_grad_sample(
    x: torch.Tensor,
    backprops: torch.Tensor,
    kernel_size: Tuple[int, int],
    stride: Tuple[int, int],
    padding: Tuple[int, int, int, int],
    dilation: Tuple[int, int],
    groups: int,
    scale: float = 1.0,
    want_sumsq: bool = True,
    norm_only: bool = False,
    out_dtype: Optional[torch.dtype] = None,
) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Per-sample weight gradients ``[n, O, C/groups, KH, KW]`` of a 2-d convolution
    (in ``out_dtype``, by default the backprops' dtype).

    ``padding`` is ``(top, bottom, left, right)``; ``backprops`` is ``[n, O, OH, OW]``.
    ``norm_only``: the gradient tiles are formed and squared but never stored; returns
    ``(None, sumsq)``.
    """
    dev = _need_gpu(x, backprops)
    if x.dtype != backprops.dtype:
        x = x.to(backprops.dtype)
    n, C, H, W = x.shape
    O = backprops.shape[1]
    KH, KW = kernel_size
    want_sumsq = want_sumsq or norm_only
    gs = None if norm_only else torch.empty((n, O, C // groups, KH, KW), dtype=out_dtype or backprops.dtype, device=dev)
    sumsq = torch.empty((n,), dtype=torch.float32, device=dev) if want_sumsq else None
    if n == 0:
        return gs, sumsq
    x = _dense(x)
    b = _dense(backprops)
    L = lib()
    oh = (H + padding[0] + padding[1] - (dilation[0] * (KH - 1) + 1)) // stride[0] + 1
    ow = (W + padding[2] + padding[3] - (dilation[1] * (KW - 1) + 1)) // stride[1] + 1
    if b.numel() != n * O * oh * ow:
        raise ValueError(
            f"backprops {tuple(backprops.shape)} do not match the output geometry [{n},{O},{oh},{ow}]"
        )
    ws, wsb = _ws(L.dpk_conv2d_gs_workspace_bytes(n, C, O, KH, KW, groups, oh * ow), dev)
    with _timed("conv2d_gs", dev):
        check(
            "dpk_conv2d_gs",
            L.dpk_conv2d_gs(
                _ptr(x), _ptr(b), _code(b), _ptr(gs), _code(out_dtype or b.dtype), _ptr(sumsq), n, C, H, W, O, KH, KW,
                stride[0], stride[1], padding[0], padding[1], padding[2], padding[3], dilation[0],
                dilation[1], groups, float(scale), _ptr(ws), wsb, _stream(dev),
            ),
        )
    return gs, sumsq


def conv3d_grad_sample(
    x: torch.Tensor,
    backprops: torch.Tensor,
    kernel_size: Tuple[int, int, int],
    stride: Tuple[int, int, int],
    padding: Tuple[Tuple[int, int], Tuple[int, int], Tuple[int, int]],
    dilation: Tuple[int, int, int],
    groups: int,
    scale: float = 1.0,
    want_sumsq: bool = True,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Per-sample weight gradients ``[n, O, C/groups, KD, KH, KW]`` of a 3-d convolution.

    ``padding`` is ``((front, back), (top, bottom), (left, right))``; ``backprops`` is
    ``[n, O, OD, OH, OW]``.
    """
    dev = _need_gpu(x, backprops)
    if x.dtype != backprops.dtype:
        x = x.to(backprops.dtype)
    n, C, D, H, W = x.shape
    O = backprops.shape[1]
    gs = torch.empty((n, O, C // groups, *kernel_size), dtype=backprops.dtype, device=dev)
    sumsq = torch.empty((n,), dtype=torch.float32, device=dev) if want_sumsq else None
    if n == 0:
        return gs, sumsq
    x = _dense(x)
    b = _dense(backprops)
    out = [
        (size + lo + hi - (dil * (k - 1) + 1)) // st + 1
        for size, (lo, hi), dil, k, st in zip((D, H, W), padding, dilation, kernel_size, stride)
    ]
    if b.numel() != n * O * out[0] * out[1] * out[2]:
        raise ValueError(f"backprops {tuple(backprops.shape)} do not match the output geometry [{n},{O},{out}]")
    arr = lambda v: (ctypes.c_int64 * 3)(*[int(e) for e in v])  # noqa: E731
    L = lib()
    ws, wsb = _ws(L.dpk_conv3d_gs_workspace_bytes(n, C, O, *kernel_size, groups, out[0] * out[1] * out[2]), dev)
    with _timed("conv3d_gs", dev):
        check(
            "dpk_conv3d_gs",
            L.dpk_conv3d_gs(
                _ptr(x), _ptr(b), _code(b), _ptr(gs), _code(gs), _ptr(sumsq), n, C, D, H, W, O, arr(kernel_size),
                arr(stride), arr([p[0] for p in padding]), arr([p[1] for p in padding]), arr(dilation), groups,
                float(scale), _ptr(ws), wsb, _stream(dev),
            ),
        )
    return gs, sumsq


def conv_bias_grad_sample(backprops: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """``gs[n,o] = scale * sum over the spatial dims of b[n,o,...]``; its per-sample sum of
    squares rides on the result for the optimizer."""
    dev = _need_gpu(backprops)
    n, O = backprops.shape[0], backprops.shape[1]
    gs = torch.empty((n, O), dtype=backprops.dtype, device=dev)
    if n == 0:
        return gs
    sumsq = torch.empty((n,), dtype=torch.float32, device=dev)
    b = _dense(backprops).reshape(n, O, -1)
    with _timed("conv_bias_gs", dev):
        check(
            "dpk_conv_bias_gs",
            lib().dpk_conv_bias_gs(
                _ptr(b), _code(b), _ptr(gs), _code(gs), _ptr(sumsq), n, O, b.shape[2], float(scale), _stream(dev)
            ),
        )
    return _with_sumsq(gs, sumsq)


# ---- nn.Embedding -------------------------------------------------------------------
def _ids_2d(ids: torch.Tensor) -> torch.Tensor:
    if ids.dtype != torch.int64:
        ids = ids.to(torch.int64)
    return _dense(ids).reshape(ids.shape[0], math.prod(ids.shape[1:]))  # explicit: -1 is ambiguous for an empty batch


def embedding_unique_pairs(ids: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(unique_pairs [U,2], inverse [n*T])`` of the (row, id) pairs, sorted: the integer stage."""
    dev = _need_gpu(ids)
    ids2 = _ids_2d(ids)
    n, T = ids2.shape
    inverse = torch.empty((n * T,), dtype=torch.int64, device=dev)
    pairs = torch.empty((n * T, 2), dtype=torch.int64, device=dev)
    count = torch.zeros((1,), dtype=torch.int64, device=dev)
    if n * T == 0:
        return pairs[:0], inverse
    L = lib()
    ws, wsb = _ws(L.dpk_embedding_workspace_bytes(n, T, 0), dev)
    with _timed("embedding_unique_pairs", dev):
        check(
            "dpk_embedding_unique_pairs",
            L.dpk_embedding_unique_pairs(
                _ptr(ids2), n, T, _ptr(inverse), _ptr(pairs), _ptr(count), _ptr(ws), wsb, _stream(dev)
            ),
        )
    return pairs[: int(count.item())], inverse


# ---- index validation of the Embedding samplers --------------------------------------
# The entry points never wait for the stream. An id outside the table makes them write
# nothing for that position and raise a sticky int32 flag in device memory, one per device,
# that is read only when somebody asks. (In a training step nn.Embedding's own forward has
# already refused such ids before a sampler sees them.)
VALIDATE_EMBEDDING_INDICES = False  # True: every sampler call reads the flag back (a sync per call)
_EMB_STATUS: Dict[torch.device, torch.Tensor] = {}


def _emb_status(dev: torch.device) -> torch.Tensor:
    t = _EMB_STATUS.get(dev)
    if t is None:
        t = _EMB_STATUS[dev] = torch.zeros(1, dtype=torch.int32, device=dev)
    return t


def check_embedding_indices(device=None) -> None:
    """Raises ``IndexError`` if an Embedding / EmbeddingBag sampler call on ``device`` since the
    last check met an index outside its table (or bag offsets that do not ascend inside the
    index list), and clears the flag. Waits for the device."""
    devs = [torch.device(device)] if device is not None else list(_EMB_STATUS)
    for d in devs:
        d = torch.device("cuda", torch.cuda.current_device()) if d.type == "cuda" and d.index is None else d
        t = _EMB_STATUS.get(d)
        if t is not None and int(t.item()) != 0:
            t.zero_()
            raise IndexError(
                "an Embedding sampler met an index outside [0, num_embeddings) or EmbeddingBag offsets that are "
                "not ascending inside the index list; nothing was written for it"
            )


def embedding_grad_sample(
    ids: torch.Tensor, backprops: torch.Tensor, num_embeddings: int, scale: float = 1.0
) -> torch.Tensor:
    """``gs[n,v,:] = scale * sum_{t: ids[n,t]==v} b[n,t,:]`` as a dense ``[n, V, D]`` tensor.
    An id outside ``[0, V)`` contributes nothing; see :func:`check_embedding_indices`."""
    dev = _need_gpu(ids, backprops)
    ids2 = _ids_2d(ids)
    n, T = ids2.shape
    D = backprops.shape[-1]
    gs = torch.empty((n, num_embeddings, D), dtype=backprops.dtype, device=dev)
    if n == 0:
        return gs
    b = _dense(backprops).reshape(n, -1, D)
    if b.shape[1] != T:
        raise ValueError(f"ids {tuple(ids.shape)} and backprops {tuple(backprops.shape)} disagree")
    L = lib()
    ws, wsb = _ws(L.dpk_embedding_workspace_bytes(n, T, D), dev)
    with _timed("embedding_gs", dev):
        check(
            "dpk_embedding_gs",
            L.dpk_embedding_gs(
                _ptr(ids2), _ptr(b), _code(b), _ptr(gs), _code(gs), n, T, num_embeddings, D,
                float(scale), _ptr(_emb_status(dev)), _ptr(ws), wsb, _stream(dev),
            ),
        )
    if VALIDATE_EMBEDDING_INDICES:
        check_embedding_indices(dev)
    return gs


def embedding_weighted_sum(
    ids: torch.Tensor,
    backprops: torch.Tensor,
    coef: torch.Tensor,
    num_embeddings: int,
    scale: float = 1.0,
    out_dtype: Optional[torch.dtype] = None,
) -> torch.Tensor:
    """``out[v, :] = scale * sum_n coef[n] * sum_{t: ids[n,t]==v} b[n,t,:]`` as ``[V, D]``: the
    clip-weighted sum of an Embedding table's per-sample gradients, summed per id in fp32 over the
    whole batch in a fixed order. ``out_dtype``: the backprops' dtype (default) or float32."""
    dev = _need_gpu(ids, backprops, coef)
    if not native_dtype(backprops.dtype):
        raise TypeError(f"embedding_weighted_sum takes float32 and bfloat16, not {backprops.dtype}")
    ids2 = _ids_2d(ids)
    n, T = ids2.shape
    D = backprops.shape[-1]
    out = torch.empty((num_embeddings, D), dtype=out_dtype or backprops.dtype, device=dev)
    if n == 0 or T == 0:
        return out.zero_()
    b = _dense(backprops).reshape(n, -1, D)
    if b.shape[1] != T:
        raise ValueError(f"ids {tuple(ids.shape)} and backprops {tuple(backprops.shape)} disagree")
    c = _dense(coef.to(torch.float32)).reshape(-1)
    if c.numel() != n:
        raise ValueError(f"{c.numel()} coefficients for {n} samples")
    L = lib()
    ws, wsb = _ws(L.dpk_embedding_weighted_sum_workspace_bytes(n, T, D), dev)
    with _timed("embedding_weighted_sum", dev):
        check(
            "dpk_embedding_weighted_sum",
            L.dpk_embedding_weighted_sum(
                _ptr(ids2), _ptr(b), _code(b), _ptr(c), _ptr(out), _code(out), n, T, num_embeddings, D, float(scale),
                _ptr(_emb_status(dev)), _ptr(ws), wsb, _stream(dev),
            ),
        )
    if VALIDATE_EMBEDDING_INDICES:
        check_embedding_indices(dev)
    return out


def embedding_ghost_norm(ids: torch.Tensor, backprops: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """Per-sample norm (fp32) of the Embedding weight gradient without forming it."""
    dev = _need_gpu(ids, backprops)
    ids2 = _ids_2d(ids)
    n, T = ids2.shape
    D = backprops.shape[-1]
    norm = torch.empty((n,), dtype=torch.float32, device=dev)
    if n == 0:
        return norm
    b = _dense(backprops).reshape(n, -1, D)
    if b.shape[1] != T:
        raise ValueError(f"ids {tuple(ids.shape)} and backprops {tuple(backprops.shape)} disagree")
    L = lib()
    ws, wsb = _ws(L.dpk_embedding_workspace_bytes(n, T, D), dev)
    with _timed("embedding_ghost_norm", dev):
        check(
            "dpk_embedding_ghost_norm",
            L.dpk_embedding_ghost_norm(
                _ptr(ids2), _ptr(b), _code(b), _ptr(norm), n, T, D, float(scale), _ptr(ws), wsb,
                _stream(dev),
            ),
        )
    return norm


def tied_embedding_cross_term(
    ids: torch.Tensor,
    emb_backprops: torch.Tensor,
    head_activations: torch.Tensor,
    head_backprops: torch.Tensor,
    scale: float = 1.0,
) -> torch.Tensor:
    """``<G_emb, G_head>`` per sample (fp32 ``[n]``) for a weight shared by an Embedding
    (``ids`` ``[n, ...]``, output backprops ``[n, ..., D]``) and a bias-free or biased Linear
    (inputs ``[n, ..., D]``, output backprops ``[n, ..., V]``), without forming either
    gradient: ``scale * sum_t <e_t, sum_t' g[t', ids_t] a_t'>``."""
    emb_backprops, head_backprops, head_activations = widen(emb_backprops), widen(head_backprops), widen(head_activations)
    dev = _need_gpu(ids, emb_backprops, head_activations, head_backprops)
    ids2 = _ids_2d(ids)
    n, T = ids2.shape
    D, V = emb_backprops.shape[-1], head_backprops.shape[-1]
    cross = torch.empty((n,), dtype=torch.float32, device=dev)
    if n == 0:
        return cross
    e = _dense(emb_backprops).reshape(n, -1, D)
    g = _dense(head_backprops).reshape(n, -1, V)
    a = _dense(head_activations).reshape(n, -1, D)
    if a.dtype != g.dtype:
        a = a.to(g.dtype)
    T2 = g.shape[1]
    if e.shape[1] != T or a.shape[1] != T2:
        raise ValueError(
            f"ids {tuple(ids.shape)}, embedding backprops {tuple(emb_backprops.shape)}, projection inputs "
            f"{tuple(head_activations.shape)} and backprops {tuple(head_backprops.shape)} disagree"
        )
    L = lib()
    ws, wsb = _ws(L.dpk_tied_embedding_cross_workspace_bytes(n, T, T2, D, _code(g)), dev)
    with _timed("tied_embedding_cross", dev):
        check(
            "dpk_tied_embedding_cross",
            L.dpk_tied_embedding_cross(
                _ptr(ids2), _ptr(e), _code(e), _ptr(a), _ptr(g), _code(g), _ptr(cross), n, T, T2, D, V,
                float(scale), _ptr(ws), wsb, _stream(dev),
            ),
        )
    return cross


def embedding_bag_grad_sample(
    index: torch.Tensor,
    offsets: torch.Tensor,
    backprops: torch.Tensor,
    num_embeddings: int,
    mode: str = "sum",
    scale: float = 1.0,
) -> torch.Tensor:
    """Per-sample gradient ``[bags, V, D]`` of ``nn.EmbeddingBag``: every index of bag ``i``
    receives ``backprops[i]`` (``/ len(bag)`` for ``mode="mean"``) once."""
    dev = _need_gpu(index, offsets, backprops)
    if mode not in ("sum", "mean"):
        raise NotImplementedError(f"EmbeddingBag mode {mode!r}: only 'sum' and 'mean' have per-sample gradients")
    if index.dtype != torch.int64 or offsets.dtype != torch.int64:
        raise TypeError("EmbeddingBag indices and offsets must be int64")
    nbags, D = offsets.shape[0], backprops.shape[-1]
    if backprops.shape[0] != nbags:
        raise ValueError(f"{nbags} bags but backprops of shape {tuple(backprops.shape)}")
    idx, off, b = _dense(index).reshape(-1), _dense(offsets), _dense(backprops).reshape(nbags, D)
    gs = torch.empty((nbags, num_embeddings, D), dtype=b.dtype, device=dev)
    if nbags == 0:
        return gs
    L = lib()
    with _timed("embedding_bag_gs", dev):
        check(
            "dpk_embedding_bag_gs",
            L.dpk_embedding_bag_gs(
                _ptr(idx), _ptr(off), _ptr(b), _code(b), _ptr(gs), _code(gs), nbags, idx.numel(), num_embeddings, D,
                int(mode == "mean"), float(scale), _ptr(_emb_status(dev)), _stream(dev),
            ),
        )
    if VALIDATE_EMBEDDING_INDICES:
        check_embedding_indices(dev)
    return gs


# ---- normalisation layers -----------------------------------------------------------
def group_norm_grad_sample(
    x: torch.Tensor,
    backprops: torch.Tensor,
    num_groups: int,
    eps: float,
    scale: float = 1.0,
    want_weight: bool = True,
    want_bias: bool = True,
) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Per-sample gradients ``[n, C]`` of GroupNorm's weight and bias, each with its per-sample sum
    of squares riding on it for the optimizer."""
    dev = _need_gpu(x, backprops)
    if x.dtype != backprops.dtype:
        x = x.to(backprops.dtype)
    n, C = x.shape[0], x.shape[1]
    gw = torch.empty((n, C), dtype=backprops.dtype, device=dev) if want_weight else None
    gb = torch.empty((n, C), dtype=backprops.dtype, device=dev) if want_bias else None
    if n == 0 or not (want_weight or want_bias):
        return gw, gb
    xd = _dense(x).reshape(n, C, -1)
    bd = _dense(backprops).reshape(n, C, -1)
    ssw = torch.empty((n,), dtype=torch.float32, device=dev) if want_weight else None
    ssb = torch.empty((n,), dtype=torch.float32, device=dev) if want_bias else None
    with _timed("group_norm_gs", dev):
        check(
            "dpk_group_norm_gs",
            lib().dpk_group_norm_gs(
                _ptr(xd), _ptr(bd), _code(bd), _ptr(gw), _ptr(gb), _code(backprops.dtype), _ptr(ssw), _ptr(ssb),
                n, C, xd.shape[2], num_groups, float(eps), float(scale), _stream(dev),
            ),
        )
    return (_with_sumsq(gw, ssw) if want_weight else None), (_with_sumsq(gb, ssb) if want_bias else None)


def rms_norm_grad_sample(
    x: torch.Tensor, backprops: torch.Tensor, normalized_numel: int, eps: float, scale: float = 1.0
) -> torch.Tensor:
    """Per-sample gradient ``[n, D]`` of RMSNorm's weight (``D = normalized_numel``); its
    per-sample sum of squares rides on the result for the optimizer."""
    dev = _need_gpu(x, backprops)
    if x.dtype != backprops.dtype:
        x = x.to(backprops.dtype)
    n, D = x.shape[0], normalized_numel
    gw = torch.empty((n, D), dtype=backprops.dtype, device=dev)
    if n == 0:
        return gw
    sumsq = torch.empty((n,), dtype=torch.float32, device=dev)
    xd = _dense(x).reshape(n, -1, D)
    bd = _dense(backprops).reshape(n, -1, D)
    T = xd.shape[1]
    L = lib()
    ws, wsb = _ws(L.dpk_rms_norm_gs_workspace_bytes(n, T, D), dev)
    with _timed("rms_norm_gs", dev):
        check(
            "dpk_rms_norm_gs",
            L.dpk_rms_norm_gs(
                _ptr(xd), _ptr(bd), _code(bd), _ptr(gw), _code(gw), _ptr(sumsq), n, T, D, float(eps), float(scale),
                _ptr(ws), wsb, _stream(dev),
            ),
        )
    return _with_sumsq(gw, sumsq)


def layer_norm_grad_sample(
    x: torch.Tensor,
    backprops: torch.Tensor,
    normalized_numel: int,
    eps: float,
    scale: float = 1.0,
    want_weight: bool = True,
    want_bias: bool = True,
) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Per-sample gradients ``[n, D]`` of LayerNorm's weight and bias (``D = normalized_numel``),
    each with its per-sample sum of squares riding on it for the optimizer."""
    dev = _need_gpu(x, backprops)
    if x.dtype != backprops.dtype:
        x = x.to(backprops.dtype)
    n, D = x.shape[0], normalized_numel
    gw = torch.empty((n, D), dtype=backprops.dtype, device=dev) if want_weight else None
    gb = torch.empty((n, D), dtype=backprops.dtype, device=dev) if want_bias else None
    if n == 0 or not (want_weight or want_bias):
        return gw, gb
    xd = _dense(x).reshape(n, -1, D)
    bd = _dense(backprops).reshape(n, -1, D)
    T = xd.shape[1]
    L = lib()
    ssw = torch.empty((n,), dtype=torch.float32, device=dev) if want_weight else None
    ssb = torch.empty((n,), dtype=torch.float32, device=dev) if want_bias else None
    ws, wsb = _ws(L.dpk_layer_norm_gs_workspace_bytes(n, T, D), dev)
    with _timed("layer_norm_gs", dev):
        check(
            "dpk_layer_norm_gs",
            L.dpk_layer_norm_gs(
                _ptr(xd), _ptr(bd), _code(bd), _ptr(gw), _ptr(gb), _code(bd), _ptr(ssw), _ptr(ssb), n, T, D,
                float(eps), float(scale), _ptr(ws), wsb, _stream(dev),
            ),
        )
    return (_with_sumsq(gw, ssw) if want_weight else None), (_with_sumsq(gb, ssb) if want_bias else None)


# ---- optimizer: norms, clip factor, clip-weighted sum, noise ---------------------------
def _flat2d(gs: torch.Tensor) -> torch.Tensor:
    g = _dense(gs)
    return g.reshape(g.shape[0], math.prod(g.shape[1:]))  # explicit: -1 is ambiguous for an empty batch


def sumsq_rows(gs_list: Sequence[torch.Tensor]) -> torch.Tensor:
    """``out[k, i] = sum of squares of sample i of tensor k`` (fp32), one pass over each tensor."""
    if _any_half(gs_list):
        gs_list = [widen(g) for g in gs_list]
    dev = _need_gpu(*gs_list)
    K = len(gs_list)
    n = gs_list[0].shape[0]
    out = torch.empty((K, n), dtype=torch.float32, device=dev)
    if n == 0 or K == 0:
        return out
    flats = [_flat2d(g) for g in gs_list]
    dt = flats[0].dtype
    if any(f.dtype != dt or f.shape[0] != n for f in flats):
        raise ValueError("per-sample gradient tensors must share the batch size and dtype")
    L = lib()
    for lo in range(0, K, DPK_MULTI_MAX):
        chunk = flats[lo : lo + DPK_MULTI_MAX]
        k = len(chunk)
        ptrs = (ctypes.c_void_p * k)(*[f.data_ptr() for f in chunk])
        sizes = (ctypes.c_int64 * k)(*[f.shape[1] for f in chunk])
        ws, wsb = _ws(L.dpk_sumsq_rows_multi_workspace_bytes(n, sizes, k), dev)
        with _timed("sumsq_rows", dev):
            check(
                "dpk_sumsq_rows_multi",
                L.dpk_sumsq_rows_multi(
                    ptrs, sizes, k, _code(dt), n, _ptr(out[lo : lo + k]), _ptr(ws), wsb, _stream(dev)
                ),
            )
    return out


def clip_factor(
    values: torch.Tensor, max_grad_norm: float, is_norm: bool = False
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(norm[n], clip[n])`` from ``values[K, n]`` (squared norms, or norms with ``is_norm``)."""
    dev = _need_gpu(values)
    v = _dense(values.to(torch.float32)).reshape(math.prod(values.shape[:-1]), values.shape[-1])
    K, n = v.shape
    norm = torch.empty((n,), dtype=torch.float32, device=dev)
    clip = torch.empty((n,), dtype=torch.float32, device=dev)
    if n == 0:
        return norm, clip
    check(
        "dpk_clip_factor",
        lib().dpk_clip_factor(
            _ptr(v), K, n, int(is_norm), float(max_grad_norm), _ptr(norm), _ptr(clip), _stream(dev)
        ),
    )
    return norm, clip


def clip_factor_per_layer(
    values: torch.Tensor, max_grad_norms: Sequence[float], is_norm: bool = False
) -> torch.Tensor:
    """``clip[K, n]`` with ``clip[k] = min(1, C_k / (norm_k + 1e-6))`` from ``values[K, n]``
    (squared norms, or norms with ``is_norm``)."""
    dev = _need_gpu(values)
    v = _dense(values.to(torch.float32)).reshape(math.prod(values.shape[:-1]), values.shape[-1])
    K, n = v.shape
    if len(max_grad_norms) != K:
        raise ValueError(f"{len(max_grad_norms)} bounds for {K} parameters")
    clip = torch.empty((K, n), dtype=torch.float32, device=dev)
    if n == 0:
        return clip
    L = lib()
    for lo in range(0, K, DPK_MULTI_MAX):
        k = min(DPK_MULTI_MAX, K - lo)
        bounds = (ctypes.c_float * k)(*[float(c) for c in max_grad_norms[lo : lo + k]])
        check(
            "dpk_clip_factor_per_layer",
            L.dpk_clip_factor_per_layer(_ptr(v[lo:]), k, n, int(is_norm), bounds, _ptr(clip[lo:]), _stream(dev)),
        )
    return clip


def clip_accumulate(
    gs_list: Sequence[torch.Tensor],
    clip: torch.Tensor,
    summed_list: Sequence[torch.Tensor],
    accumulate: bool,
) -> None:
    """``summed_k (+)= sum_n clip[n] * gs_k[n]`` for every k, reading each gs once. ``clip`` is
    one vector ``[n]`` for all tensors, or a table ``[K, n]`` with a row per tensor."""
    if _any_half(gs_list, summed_list):
        wide = [widen(s_) for s_ in summed_list]
        clip_accumulate([widen(g) for g in gs_list], clip, wide, accumulate)
        _narrow_back(summed_list, wide)
        return
    dev = _need_gpu(clip, *gs_list, *summed_list)
    K = len(gs_list)
    if K == 0:
        return
    n = gs_list[0].shape[0]
    per_layer = clip.dim() == 2
    flats = [_flat2d(g) for g in gs_list]
    gdt, odt = flats[0].dtype, summed_list[0].dtype
    for f, s in zip(flats, summed_list):
        if f.dtype != gdt or s.dtype != odt or f.shape[0] != n:
            raise ValueError("tensors of one clip_accumulate call must share batch size and dtypes")
        if not s.is_contiguous() or s.numel() != f.shape[1]:
            raise ValueError("summed tensors must be dense and match the per-sample gradient size")
    if clip.dtype != torch.float32 or clip.shape != ((K, n) if per_layer else (n,)):
        raise ValueError("clip must be float32 of shape [n], or [K, n] with a row per tensor")
    clip = _dense(clip)
    L = lib()
    name = "dpk_clip_accumulate_per_layer" if per_layer else "dpk_clip_accumulate_multi"
    fn = getattr(L, name)
    for lo in range(0, K, DPK_MULTI_MAX):
        fs, ss = flats[lo : lo + DPK_MULTI_MAX], summed_list[lo : lo + DPK_MULTI_MAX]
        k = len(fs)
        gptrs = (ctypes.c_void_p * k)(*[f.data_ptr() for f in fs])
        sptrs = (ctypes.c_void_p * k)(*[s.data_ptr() for s in ss])
        sizes = (ctypes.c_int64 * k)(*[f.shape[1] for f in fs])
        factors = clip[lo:] if per_layer else clip
        with _timed("clip_accumulate", dev):
            check(
                name,
                fn(gptrs, sptrs, sizes, k, _code(gdt), _code(odt), _ptr(factors), n, int(accumulate), _stream(dev)),
            )


def add_noise(
    summed: torch.Tensor,
    grad: torch.Tensor,
    std: float,
    denom: float,
    seed: int,
    offset: int,
    draws: int = 1,
) -> None:
    """``grad = (summed + std * z) / denom`` with ``z ~ N(0,1)`` from Philox(seed, offset)."""
    if _any_half((summed, grad)):
        wide = widen(grad)
        add_noise(widen(summed), wide, std, denom, seed, offset, draws)
        _narrow_back((grad,), (wide,))
        return
    dev = _need_gpu(summed, grad)
    if not summed.is_contiguous() or not grad.is_contiguous() or summed.numel() != grad.numel():
        raise ValueError("summed and grad must be dense and of equal size")
    with _timed("add_noise", dev):
        check(
            "dpk_add_noise",
            lib().dpk_add_noise(
                _ptr(summed), _code(summed), _ptr(grad), _code(grad), summed.numel(), float(std),
                float(denom), seed & 0xFFFFFFFFFFFFFFFF, offset & 0xFFFFFFFFFFFFFFFF, draws, _stream(dev),
            ),
        )


def add_noise_multi(
    summed_list: Sequence[torch.Tensor],
    grad_list: Sequence[torch.Tensor],
    std: float,
    denom: float,
    seed: int,
    offset: int,
    draws: int = 1,
) -> int:
    """``grad_k = (summed_k + std * z) / denom`` for every k; one Philox stream laid across the
    tensors in order, one launch per ``DPK_MULTI_MAX`` tensors. Returns the number of offset units
    consumed (``draws`` per launch), by which the caller advances its generator."""
    K = len(summed_list)
    if K == 0:
        return 0
    if _any_half(summed_list, grad_list):
        wide = [widen(g) for g in grad_list]
        used = add_noise_multi([widen(s_) for s_ in summed_list], wide, std, denom, seed, offset, draws)
        _narrow_back(grad_list, wide)
        return used
    dev = _need_gpu(*summed_list, *grad_list)
    idt, odt = summed_list[0].dtype, grad_list[0].dtype
    for s, g in zip(summed_list, grad_list):
        if s.dtype != idt or g.dtype != odt:
            raise ValueError("tensors of one add_noise_multi call must share dtypes")
        if not s.is_contiguous() or not g.is_contiguous() or s.numel() != g.numel():
            raise ValueError("summed and grad tensors must be dense and of equal size")
    L = lib()
    used = 0
    for lo in range(0, K, DPK_MULTI_MAX):
        ss, gg = summed_list[lo : lo + DPK_MULTI_MAX], grad_list[lo : lo + DPK_MULTI_MAX]
        k = len(ss)
        sptrs = (ctypes.c_void_p * k)(*[t.data_ptr() for t in ss])
        gptrs = (ctypes.c_void_p * k)(*[t.data_ptr() for t in gg])
        sizes = (ctypes.c_int64 * k)(*[t.numel() for t in ss])
        with _timed("add_noise", dev):
            check(
                "dpk_add_noise_multi",
                L.dpk_add_noise_multi(
                    sptrs, gptrs, sizes, k, _code(idt), _code(odt), float(std), float(denom),
                    seed & 0xFFFFFFFFFFFFFFFF, (offset + used) & 0xFFFFFFFFFFFFFFFF, draws,
                    _stream(dev),
                ),
            )
        used += draws
    return used


CLIP_NOISE_STEP_MIN_N, CLIP_NOISE_STEP_MAX_N = 64, 1024


def clip_noise_step(
    gs_list: Sequence[torch.Tensor],
    sumsq_list: Sequence[torch.Tensor],
    grad_list: Sequence[torch.Tensor],
    summed_list: Optional[Sequence[torch.Tensor]],
    max_grad_norm: float,
    std: float,
    denom: float,
    seed: int,
    offset: int,
    draws: int = 1,
) -> None:
    """The whole step of a small model in one launch: clip factors from the per-parameter squared
    norms ``sumsq_list`` (``float32[n]`` each), ``summed_k = sum_n clip[n] * gs_k[n]`` (stored when
    ``summed_list`` is given) and ``grad_k = (summed_k + std * z) / denom`` with the noise stream of
    :func:`add_noise_multi`. At most ``DPK_MULTI_MAX`` tensors of 64 to 1024 samples; the results
    are the bits that :func:`clip_factor`, :func:`clip_accumulate` and :func:`add_noise_multi` give."""
    K = len(gs_list)
    dev = _need_gpu(*gs_list, *sumsq_list, *grad_list)
    n = gs_list[0].shape[0]
    gdt, odt = gs_list[0].dtype, grad_list[0].dtype
    gptrs = (ctypes.c_void_p * K)(*[t.data_ptr() for t in gs_list])
    qptrs = (ctypes.c_void_p * K)(*[t.data_ptr() for t in sumsq_list])
    optrs = (ctypes.c_void_p * K)(*[t.data_ptr() for t in grad_list])
    sptrs = (ctypes.c_void_p * K)(*[t.data_ptr() for t in summed_list]) if summed_list is not None else None
    sizes = (ctypes.c_int64 * K)(*[t.numel() for t in grad_list])
    with _timed("clip_noise_step", dev):
        check(
            "dpk_clip_noise_step",
            lib().dpk_clip_noise_step(
                gptrs, qptrs, optrs, sptrs, sizes, K, _code(gdt), _code(odt), n, float(max_grad_norm), float(std),
                float(denom), seed & 0xFFFFFFFFFFFFFFFF, offset & 0xFFFFFFFFFFFFFFFF, draws, _stream(dev),
            ),
        )


def fill_normal(out: torch.Tensor, std: float, seed: int, offset: int) -> None:
    dev = _need_gpu(out)
    if out.dtype != torch.float32 or not out.is_contiguous():
        raise ValueError("fill_normal needs a dense float32 tensor")
    check(
        "dpk_fill_normal",
        lib().dpk_fill_normal(
            _ptr(out), out.numel(), float(std), seed & 0xFFFFFFFFFFFFFFFF, offset & 0xFFFFFFFFFFFFFFFF,
            _stream(dev),
        ),
    )


def device_cus() -> int:
    return lib().dpk_device_cus()
