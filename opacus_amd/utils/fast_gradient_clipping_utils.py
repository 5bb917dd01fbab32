"""Loss wrappers that fold ghost clipping's two backward passes into ``loss.backward()``.

Mirror of opacus/utils/fast_gradient_clipping_utils.py.
"""

from __future__ import annotations

import copy
import warnings

import torch


def first_pass_backward(module, reduced: torch.Tensor, retain_graph: bool = True) -> None:
    """Backward pass #1 of ghost clipping (fast_gradient_clipping_utils.py:189): only there
    to let the hooks see the gradients of the layers' outputs. When the module can name the
    tensors at the start of the graph, autograd is asked for those alone, which leaves out
    the weight-gradient GEMMs of the pass; what they would have written to ``.grad`` is
    zeroed by the caller in the next line anyway."""
    leaves = getattr(module, "first_backward_inputs", None)
    inputs = leaves() if callable(leaves) else None
    if isinstance(inputs, (list, tuple)) and len(inputs) > 0:
        # autograd.grad rather than backward(inputs=...): the gradients of these tensors are only
        # wanted by the hooks on the way, and backward() would clone each of them into ``.grad``
        # (for an activation at the start of a large model that is a copy of hundreds of MB)
        torch.autograd.grad(reduced, list(inputs), retain_graph=retain_graph, allow_unused=True)
    else:
        reduced.backward(retain_graph=retain_graph)


_warned_two_passes = False


def _warn_two_passes_once() -> None:
    global _warned_two_passes
    if not _warned_two_passes:
        _warned_two_passes = True
        warnings.warn(
            "The loss depends on trainable parameters other than through the layers that ghost clipping "
            "hooks (a regulariser on the weights, a functional use of a layer's weight, a layer that uses "
            "a parameter more than once per call): such steps run the two backward passes of the reference "
            "instead of the single pass. Pass single_backward=False to silence this warning.",
            stacklevel=3,
        )


class DPTensorFastGradientClipping:
    """A per-sample loss bound to its module and optimizer. ``backward()`` runs: backward #1
    (hooks collect per-sample gradient norms), ``optimizer.zero_grad()``, clipping
    coefficients, hooks off, backward #2 of ``sum_n coef[n] * loss[n]`` (which leaves the
    clipped gradient sum in ``p.grad``), hooks on (fast_gradient_clipping_utils.py:179-201).
    A module built with ``single_backward=True`` forms that sum from the first pass instead."""

    def __init__(self, module, optimizer, loss_per_sample: torch.Tensor, loss_reduction: str = "mean"):
        self.module = module
        self.optimizer = optimizer
        self.loss_per_sample = loss_per_sample
        self.loss_reduction = loss_reduction

    def _like(self, loss_per_sample: torch.Tensor) -> "DPTensorFastGradientClipping":
        # a shallow copy, so that subclasses keep their own settings
        new = copy.copy(self)
        new.loss_per_sample = loss_per_sample
        return new

    def _other(self, other):
        if isinstance(other, DPTensorFastGradientClipping):
            if other.loss_reduction != self.loss_reduction:
                raise ValueError(
                    f"Cannot combine losses with different reductions: {self.loss_reduction} vs {other.loss_reduction}"
                )
            return other.loss_per_sample
        return other

    def item(self):
        return self.detach().item()

    def detach(self):
        if self.loss_reduction == "mean":
            return torch.mean(self.loss_per_sample).detach()
        if self.loss_reduction == "sum":
            return torch.sum(self.loss_per_sample).detach()

    # arithmetic keeps the binding to module and optimizer (:60-169)
    def __truediv__(self, other):
        return self._like(self.loss_per_sample / other)

    def __mul__(self, other):
        return self._like(self.loss_per_sample * other)

    def __rmul__(self, other):
        return self.__mul__(other)

    def __add__(self, other):
        return self._like(self.loss_per_sample + self._other(other))

    def __radd__(self, other):
        return self.__add__(other)

    def __sub__(self, other):
        return self._like(self.loss_per_sample - self._other(other))

    def __rsub__(self, other):
        return self._like(other - self.loss_per_sample)

    def __neg__(self):
        return self._like(-self.loss_per_sample)

    def __repr__(self):
        return f"DPTensorFastGradientClipping(loss_reduction={self.loss_reduction}, shape={self.loss_per_sample.shape})"

    def __str__(self):
        return f"DPTensorFastGradientClipping({self.item():.4f})"

    def backward(self):
        if self.loss_reduction == "mean":
            reduced = torch.mean(self.loss_per_sample, dim=0)
        elif self.loss_reduction == "sum":
            reduced = torch.sum(self.loss_per_sample, dim=0)
        else:
            raise ValueError(f"loss_reduction = {self.loss_reduction}. Only 'sum' and 'mean' losses are supported")
        single = getattr(self.module, "single_backward", False) is True
        if single and not self.module.single_pass_is_exact(reduced):
            # the loss reaches a trainable parameter other than through a hooked layer: only
            # autograd's second pass differentiates that term, so this step takes both passes
            _warn_two_passes_once()
            self.module.single_backward = False
            try:
                self._backward(reduced, single=False)
            finally:
                self.module.single_backward = True
            return
        self._backward(reduced, single)

    def _backward(self, reduced: torch.Tensor, single: bool) -> None:
        first_pass_backward(self.module, reduced, retain_graph=not single)
        self.optimizer.zero_grad()
        coeff = self.module.get_clipping_coef()
        if single:
            # the clipped sum straight from what the hooks kept of the first pass
            self.module.accumulate_clipped_gradients(coeff)
            return
        weighted = coeff.to(self.loss_per_sample.device) * self.loss_per_sample
        second_loss = torch.sum(weighted)
        self.module.disable_hooks()
        second_loss.backward()
        self.module.enable_hooks()


class DPLossFastGradientClipping:
    """Wraps a criterion so that calling it yields a :class:`DPTensorFastGradientClipping`
    holding the per-sample loss (fast_gradient_clipping_utils.py:204-276)."""

    def __init__(self, module, optimizer, criterion, loss_reduction: str = "mean"):
        assert loss_reduction in ["mean", "sum"], "loss_reduction should be either 'mean' or 'sum'"
        if not hasattr(criterion, "reduction"):
            setattr(criterion, "reduction", module.loss_reduction)
        assert (
            loss_reduction == criterion.reduction == module.loss_reduction == optimizer.loss_reduction
        ), "loss_reduction should be the same across GradSampleModule, Optimizer, Criterion, and loss_reduction"
        self.optimizer = optimizer
        self.module = module
        self.criterion = criterion
        self.loss_reduction = loss_reduction

    def __call__(self, *args, shape=None, **kwargs) -> DPTensorFastGradientClipping:
        saved = self.criterion.reduction
        self.criterion.reduction = "none"
        try:
            loss_per_sample = self.criterion(*args, **kwargs)
        finally:
            self.criterion.reduction = saved
        if shape is not None and loss_per_sample.shape[0] == shape[0] * shape[1]:
            # token-level losses of a [batch, seq, ...] model: one loss per sequence, since the
            # sequence is the privacy unit (:248-272)
            per_token = loss_per_sample.view(shape[0], shape[1])
            if self.loss_reduction == "mean":
                ignore_index = getattr(self.criterion, "ignore_index", None)
                if ignore_index is not None and len(args) >= 2:
                    targets = kwargs["target"] if "target" in kwargs else args[1]
                    valid = (targets.view(shape[0], shape[1]) != ignore_index).sum(dim=1).clamp(min=1)
                    loss_per_sample = per_token.sum(dim=1) / valid
                else:
                    loss_per_sample = per_token.mean(dim=1)
            elif self.loss_reduction == "sum":
                loss_per_sample = per_token.sum(dim=1)
            else:
                raise ValueError(f"loss_reduction = {self.loss_reduction}. Only 'sum' and 'mean' losses are supported")
        return DPTensorFastGradientClipping(self.module, self.optimizer, loss_per_sample, self.loss_reduction)
