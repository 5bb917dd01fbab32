"""Base classes of the per-sample-gradient engine (mirror of opacus/grad_sample/gsm_base.py).

A hooks object attaches to a module and gives every trainable parameter the extra
attributes ``grad_sample`` and ``_forward_counter``; the ``nn.Module`` flavour also
wraps the module so that ``forward``, ``state_dict`` (keys prefixed ``_module.``) and
submodule attribute access keep working.
"""

from __future__ import annotations

import logging
from abc import ABC, abstractmethod

import torch.nn as nn

from ..utils.module_utils import trainable_parameters

logger = logging.getLogger(__name__)

# Attributes this package hangs on parameters; ``cleanup`` removes all of them.
OPACUS_PARAM_MONKEYPATCH_ATTRS = ["grad_sample", "_forward_counter", "_current_grad_sample", "_norm_sample"]


class AbstractGradSampleHooks(ABC):
    """State shared by every hooks flavour (opacus/grad_sample/gsm_base.py:35-128)."""

    def __init__(self, m: nn.Module, *, batch_first=True, loss_reduction="mean"):
        super().__init__()
        self._module = m
        self.batch_first = batch_first
        self.loss_reduction = loss_reduction
        for _, p in trainable_parameters(self._module):
            p.grad_sample = None
            p._forward_counter = 0

    def set_grad_sample_to_none(self):
        for p in self._module.parameters():
            p.grad_sample = None

    def del_grad_sample(self):
        for p in self._module.parameters():
            del p.grad_sample

    def forbid_grad_accumulation(self):
        """After this, a second backward pass without ``zero_grad`` must raise (no-op here)."""

    def allow_grad_accumulation(self):
        """Undoes :meth:`forbid_grad_accumulation` (no-op here)."""

    @abstractmethod
    def remove_hooks(self) -> None:
        ...

    def cleanup(self):
        """Removes the hooks and every attribute this package added to the parameters."""
        try:
            self.remove_hooks()
        except Exception as e:  # still strip the attributes
            logger.warning(f"Failed to remove hooks during cleanup: {e}. Attempting to clean up attributes anyway.")
        finally:
            for p in self._module.parameters():
                for attr in OPACUS_PARAM_MONKEYPATCH_ATTRS:
                    if hasattr(p, attr):
                        delattr(p, attr)


class AbstractGradSampleModule(nn.Module, AbstractGradSampleHooks, ABC):
    """``nn.Module`` wrapper flavour (opacus/grad_sample/gsm_base.py:131-221)."""

    def __init__(self, m: nn.Module, *, batch_first=True, loss_reduction="mean"):
        nn.Module.__init__(self)
        AbstractGradSampleHooks.__init__(self, m, batch_first=batch_first, loss_reduction=loss_reduction)
        self.grad_accumulation_hook = None

    def forward(self, *args, **kwargs):
        return self._module(*args, **kwargs)

    def __getattr__(self, item):
        try:
            return super().__getattr__(item)
        except AttributeError as e:
            # let `wrapped.fc1` reach the wrapped module's submodules
            submodules = dict(self._module.named_modules())
            if item and item in submodules:
                return submodules[item]
            raise e

    def zero_grad(self, set_to_none: bool = False):
        """Clears ``p.grad`` as usual and always sets ``p.grad_sample`` to None."""
        self.set_grad_sample_to_none()
        super().zero_grad(set_to_none)

    def to_standard_module(self) -> nn.Module:
        """The wrapped module with hooks and per-sample attributes removed."""
        self._close()
        return self._module

    def _close(self):
        self.cleanup()

    def __repr__(self):
        return f"{type(self).__name__}({self._module.__repr__()})"
