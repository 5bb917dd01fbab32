"""Per-layer clipping (mirror of opacus/optimizers/perlayeroptimizer.py).

Every parameter tensor has a clipping bound of its own and is clipped on its own norm. The
per-sample gradients are still read once, all parameters in one launch: the kernel takes a
``[K, n]`` table of clip factors instead of one vector.
"""

from __future__ import annotations

import math
from typing import List, Optional

import torch
from torch import nn
from torch.optim import Optimizer

from .. import kernels
from .optimizer import DPOptimizer
from .utils import params


class DPPerLayerOptimizer(DPOptimizer):
    """``max_grad_norm`` is a list with one bound per parameter; the noise is calibrated to
    their 2-norm, the sensitivity of the whole clipped gradient (perlayeroptimizer.py:32-56)."""

    def __init__(
        self,
        optimizer: Optimizer,
        *,
        noise_multiplier: float,
        max_grad_norm: List[float],
        expected_batch_size: Optional[int],
        loss_reduction: str = "mean",
        generator=None,
        secure_mode: bool = False,
        **kwargs,
    ):
        if len(max_grad_norm) != len(params(optimizer)):
            raise ValueError(
                f"per-layer clipping needs one bound per parameter: got {len(max_grad_norm)} for "
                f"{len(params(optimizer))} parameters"
            )
        self.max_grad_norms = [float(c) for c in max_grad_norm]
        super().__init__(
            optimizer,
            noise_multiplier=noise_multiplier,
            max_grad_norm=math.sqrt(sum(c * c for c in self.max_grad_norms)),
            expected_batch_size=expected_batch_size,
            loss_reduction=loss_reduction,
            generator=generator,
            secure_mode=secure_mode,
            **kwargs,
        )

    def _clip_factors(self, plist: List[nn.Parameter], flats: List[torch.Tensor]) -> torch.Tensor:
        """``clip[k, i] = min(1, C_k / (||g_k[i]|| + 1e-6))`` (perlayeroptimizer.py:62-68)."""
        n = len(flats[0])
        if n == 0:
            return torch.zeros((len(plist), 0), device=flats[0].device, dtype=torch.float32)
        sumsq = self._per_param_sumsq(plist, flats)
        return kernels.clip_factor_per_layer(sumsq, self.max_grad_norms)
