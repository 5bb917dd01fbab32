"""Ghost clipping with a clipping bound that tracks a quantile of the per-sample norms.

Mirror of opacus/utils/adaptive_clipping/adaptive_clipping_utils.py. Between the two backward
passes of ghost clipping the bound moves geometrically towards the target quantile of the
per-sample gradient norms (Andrew et al., "Differentially Private Learning with Adaptive
Clipping"), the count of unclipped samples is privatised with Gaussian noise of standard
deviation ``batch / 20``, and the gradient noise multiplier is raised so that the two
mechanisms together cost what the original multiplier would.

The per-sample norms come from the ghost-norm kernels; what is added here is arithmetic on
one ``[n]`` vector and two host scalars per step.
"""

from __future__ import annotations

import math

import torch
import torch.nn as nn

from ...privacy_engine import PrivacyEngine
from ..fast_gradient_clipping_utils import (
    DPLossFastGradientClipping,
    DPTensorFastGradientClipping,
    first_pass_backward,
)


class DPTensorFastGradientAdaptiveClipping(DPTensorFastGradientClipping):
    """``backward()`` = backward #1, per-sample norms, bound and noise-multiplier update,
    coefficients from the *new* bound, backward #2 (adaptive_clipping_utils.py:32-121)."""

    def __init__(
        self,
        module,
        optimizer,
        loss_per_sample: torch.Tensor,
        loss_reduction: str = "mean",
        target_unclipped_quantile: float = 0.5,
        min_clipbound: float = 1,
        max_clipbound: float = 1e8,
        clipbound_learning_rate: float = 0.2,
        initial_noise_multiplier: float = 1.0,
    ):
        super().__init__(module, optimizer, loss_per_sample, loss_reduction)
        self.target_unclipped_quantile = target_unclipped_quantile
        self.min_clipbound = min_clipbound
        self.max_clipbound = max_clipbound
        self.clipbound_learning_rate = clipbound_learning_rate
        self.initial_clipping_norm = self.optimizer.max_grad_norm
        self.initial_noise_multiplier = initial_noise_multiplier

    def _backward(self, reduced: torch.Tensor, single: bool) -> None:
        # (the base class's backward() reduces the loss and decides between one pass and two)
        first_pass_backward(self.module, reduced, retain_graph=not single)
        self.optimizer.zero_grad()

        per_sample_norms = self.module.get_norm_sample()
        new_max_grad_norm, new_noise_multiplier = self._update_clip_and_noise(per_sample_norms)
        # The optimizer's noise_multiplier stays what the accountant was told; only the
        # multiplier used to draw the noise changes (:95-101).
        self.module.max_grad_norm = new_max_grad_norm
        self.optimizer.max_grad_norm = new_max_grad_norm
        self.optimizer._adjusted_noise_multiplier = new_noise_multiplier

        # no 1e-6 in this variant: exactly 1 up to the bound, bound / norm beyond it (:103-108)
        coeff = torch.where(
            per_sample_norms <= new_max_grad_norm,
            torch.ones_like(per_sample_norms),
            new_max_grad_norm / per_sample_norms,
        )
        if single:  # the clipped sum straight from what the hooks kept of the first pass
            self.module.accumulate_clipped_gradients(coeff)
            return
        second_loss = torch.sum(coeff.to(self.loss_per_sample.device) * self.loss_per_sample)
        self.module.disable_hooks()
        second_loss.backward()
        self.module.enable_hooks()

    def _update_clip_and_noise(self, per_sample_norms: torch.Tensor):
        assert (
            self.module.max_grad_norm == self.optimizer.max_grad_norm
        ), "Max grad norm does not match between optimizer and model."
        current = self.module.max_grad_norm
        batch_size = len(per_sample_norms)
        unclipped_num = int((per_sample_norms <= current).sum().item())

        unclipped_num_std = batch_size / 20.0  # heuristic of the paper, section 3
        noisy_unclipped = unclipped_num + torch.normal(mean=0.0, std=unclipped_num_std, size=(1,)).item()
        unclipped_frac = noisy_unclipped / batch_size

        new_bound = current * math.exp(-self.clipbound_learning_rate * (unclipped_frac - self.target_unclipped_quantile))
        new_bound = min(max(new_bound, self.min_clipbound), self.max_clipbound)

        assert (
            batch_size > 10 * self.initial_noise_multiplier
        ), "Batch size is too small. For adaptive clipping, please use a batch size larger than 10 * noise_multiplier."
        if self.initial_noise_multiplier > 0:
            # Theorem 1 of the paper; the 2 comes from recentring the clipped/unclipped bit
            new_noise_multiplier = (
                self.initial_noise_multiplier ** (-2) - (2.0 * unclipped_num_std) ** (-2)
            ) ** (-1 / 2.0)
        else:
            new_noise_multiplier = self.initial_noise_multiplier
        return new_bound, new_noise_multiplier


class DPLossFastGradientAdaptiveClipping(DPLossFastGradientClipping):
    """Criterion wrapper whose result is a :class:`DPTensorFastGradientAdaptiveClipping`
    (adaptive_clipping_utils.py:178-227)."""

    def __init__(
        self,
        module,
        optimizer,
        criterion,
        loss_reduction: str = "mean",
        target_unclipped_quantile: float = 0.5,
        min_clipbound: float = 1,
        max_clipbound: float = 1e8,
        clipbound_learning_rate: float = 0.2,
        initial_noise_multiplier: float = 1.0,
    ):
        super().__init__(module, optimizer, criterion, loss_reduction)
        self.target_unclipped_quantile = target_unclipped_quantile
        self.min_clipbound = min_clipbound
        self.max_clipbound = max_clipbound
        self.clipbound_learning_rate = clipbound_learning_rate
        self.initial_noise_multiplier = initial_noise_multiplier

    def __call__(self, *args, **kwargs) -> DPTensorFastGradientAdaptiveClipping:
        plain = super().__call__(*args, **kwargs)
        return DPTensorFastGradientAdaptiveClipping(
            self.module,
            self.optimizer,
            plain.loss_per_sample,
            self.loss_reduction,
            self.target_unclipped_quantile,
            self.min_clipbound,
            self.max_clipbound,
            self.clipbound_learning_rate,
            self.initial_noise_multiplier,
        )


class PrivacyEngineAdaptiveClipping(PrivacyEngine):
    """``make_private(..., grad_sample_mode="ghost", target_unclipped_quantile=..., ...)``
    returns the adaptive criterion as its third element (adaptive_clipping_utils.py:230-279)."""

    def __init__(self, *, accountant: str = "prv", secure_mode: bool = False):
        super().__init__(accountant=accountant, secure_mode=secure_mode)

    def _prepare_criterion(
        self,
        *,
        module,
        optimizer,
        criterion=nn.CrossEntropyLoss(),
        loss_reduction: str = "mean",
        target_unclipped_quantile: float = 0.5,
        min_clipbound: float = 1,
        max_clipbound: float = 1e8,
        clipbound_learning_rate: float = 0.2,
        **kwargs,
    ) -> DPLossFastGradientAdaptiveClipping:
        return DPLossFastGradientAdaptiveClipping(
            module,
            optimizer,
            criterion,
            loss_reduction=loss_reduction,
            target_unclipped_quantile=target_unclipped_quantile,
            min_clipbound=min_clipbound,
            max_clipbound=max_clipbound,
            clipbound_learning_rate=clipbound_learning_rate,
            initial_noise_multiplier=optimizer.noise_multiplier,
        )
