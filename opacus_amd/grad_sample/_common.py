"""Helpers shared by the sampler functions."""

from __future__ import annotations

from typing import Optional

import torch


def tag_sumsq(gs: torch.Tensor, sumsq: Optional[torch.Tensor]) -> torch.Tensor:
    """Leaves the kernel's per-sample sum of squares on the tensor it describes.

    The optimizer's norm pass uses it instead of re-reading ``gs`` as long as the tensor's
    version counter says nobody wrote to ``gs`` since.
    """
    if sumsq is not None:
        gs._dpk_sumsq = sumsq
        gs._dpk_sumsq_version = gs._version
    return gs


def cached_sumsq(gs) -> Optional[torch.Tensor]:
    if not isinstance(gs, torch.Tensor):
        return None
    ss = getattr(gs, "_dpk_sumsq", None)
    if ss is not None and getattr(gs, "_dpk_sumsq_version", None) == gs._version and ss.shape[0] == gs.shape[0]:
        return ss
    return None
