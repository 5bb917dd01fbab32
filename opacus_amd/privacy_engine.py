"""``PrivacyEngine.make_private``: the drop-in entry (mirror of opacus/privacy_engine.py:307-475).

Only the wiring of the hot path is built: the module gets the per-sample-gradient hooks,
the optimizer becomes a ``DPOptimizer`` on the HIP kernels and, in ghost mode, the
criterion becomes a ``DPLossFastGradientClipping``. Privacy accounting (epsilon), Poisson
data loading, module surgery and checkpoints are separate, CPU-side subsystems of the
reference and are not part of this build: the step hook records what an accountant needs
(noise multiplier, sample rate, number of steps) and nothing more.
"""

from __future__ import annotations

import os
import warnings
from itertools import chain
from typing import List, Optional, Tuple, Union

import torch
from torch import nn, optim
from torch.utils.data import DataLoader

from .data_loader import DPDataLoader, switch_generator
from .grad_sample import AbstractGradSampleModule, GradSampleHooks, get_gsm_class, prepare_module
from .optimizers import DPOptimizer, get_optimizer_class
from .utils.fast_gradient_clipping_utils import DPLossFastGradientClipping


class StepRecorder:
    """Stands where the reference's accountant stands (opacus/accountants/accountant.py:69-87):
    ``history`` holds ``[noise_multiplier, sample_rate, num_steps]`` runs, the input of any
    accountant. Epsilon itself is not computed here."""

    def __init__(self):
        self.history: List[Tuple[float, float, int]] = []

    def step(self, *, noise_multiplier: float, sample_rate: float):
        if self.history and self.history[-1][0] == noise_multiplier and self.history[-1][1] == sample_rate:
            nm, sr, k = self.history.pop()
            self.history.append((nm, sr, k + 1))
        else:
            self.history.append((noise_multiplier, sample_rate, 1))

    def __len__(self):
        return sum(k for _, _, k in self.history)

    def get_optimizer_hook_fn(self, sample_rate: float):
        def hook(optim: DPOptimizer):
            # under data parallelism or accumulation one logical step spans several
            self.step(
                noise_multiplier=optim.noise_multiplier,
                sample_rate=sample_rate * optim.accumulated_iterations,
            )

        return hook

    def get_epsilon(self, delta: float, **kwargs) -> float:
        raise NotImplementedError(
            "privacy accounting is outside this build; feed `history` to an accountant of your choice"
        )


class PrivacyEngine:
    """Attaches DP-SGD to a (module, optimizer, data loader) triple (privacy_engine.py:36-98)."""

    SECURE_MODE_URANDOM_PHILOX = "urandom-philox"

    def __init__(self, *, accountant: str = "prv", secure_mode: Union[bool, str] = False):
        self.accountant = StepRecorder()
        self.accountant_mechanism = accountant
        if secure_mode is True:
            # The reference's secure mode is a cryptographically secure generator (torchcsprng) and it
            # refuses to run without one (privacy_engine.py:86-96). None is available here, so the
            # flag is refused too rather than honoured with something weaker; what this build can
            # offer instead has to be asked for by name.
            raise ImportError(
                "secure_mode=True asks for a cryptographically secure random number generator (the reference "
                "uses torchcsprng), which this build does not have. "
                f"secure_mode={self.SECURE_MODE_URANDOM_PHILOX!r} selects what it does have: noise keys and the "
                "sampling generator seeded from os.urandom (no seed reproduces them) and four summed draws per "
                "value, on statistical generators (Philox4x32-10, MT19937)."
            )
        if secure_mode not in (False, self.SECURE_MODE_URANDOM_PHILOX):
            raise ValueError(f"secure_mode must be False or {self.SECURE_MODE_URANDOM_PHILOX!r}, not {secure_mode!r}")
        self.secure_mode = bool(secure_mode)
        self.secure_rng = None
        self.dataset = None
        if self.secure_mode:
            # The reference builds a torchcsprng generator over /dev/urandom here and fails
            # without that package (privacy_engine.py:86-96). This build keeps what it can
            # deliver without it and says what it cannot: batch sampling uses a generator of
            # its own seeded from os.urandom (so no torch.manual_seed reaches it), every noise
            # launch takes a fresh Philox key and offset from os.urandom, and four draws are
            # summed and halved as the reference does against floating-point attacks.
            self.secure_rng = torch.Generator()
            self.secure_rng.manual_seed(int.from_bytes(os.urandom(8), "little") >> 1)
            warnings.warn(
                "secure_mode: noise keys and the sampling generator are seeded from os.urandom and "
                "cannot be reproduced by any seed, but the generators themselves (Philox4x32-10 on the "
                "GPU, MT19937 for batch sampling) are statistical, not cryptographically secure as the "
                "reference's torchcsprng is."
            )
        else:
            warnings.warn(
                "Secure RNG turned off. This is perfectly fine for experimentation as it allows "
                "for much faster training performance, but remember to turn it on and retrain "
                "one last time before production with ``secure_mode`` turned on."
            )

    # ---- pieces -------------------------------------------------------------------------
    def _prepare_optimizer(
        self,
        *,
        optimizer: optim.Optimizer,
        noise_multiplier: float,
        max_grad_norm: Union[float, List[float]],
        expected_batch_size: int,
        loss_reduction: str = "mean",
        distributed: bool = False,
        clipping: str = "flat",
        noise_generator=None,
        grad_sample_mode="hooks",
        **kwargs,
    ) -> DPOptimizer:
        if isinstance(optimizer, DPOptimizer):
            optimizer = optimizer.original_optimizer
        generator = self.secure_rng if self.secure_mode else noise_generator
        optim_class = get_optimizer_class(clipping=clipping, distributed=distributed, grad_sample_mode=grad_sample_mode)
        return optim_class(
            optimizer=optimizer,
            noise_multiplier=noise_multiplier,
            max_grad_norm=max_grad_norm,
            expected_batch_size=expected_batch_size,
            loss_reduction=loss_reduction,
            generator=generator,
            secure_mode=self.secure_mode,
            **kwargs,
        )

    def _prepare_data_loader(
        self, data_loader: DataLoader, *, poisson_sampling: bool, batch_first: bool = True, rand_on_empty: bool = False,
        **_unused,
    ) -> DataLoader:
        if self.dataset is None:
            self.dataset = data_loader.dataset
        elif self.dataset != data_loader.dataset:
            warnings.warn(
                f"PrivacyEngine detected new dataset object. Was: {self.dataset}, got: {data_loader.dataset}. "
                "Privacy accounting works per dataset, please initialize new PrivacyEngine if you're using "
                "different dataset."
            )
        if poisson_sampling:
            # privacy_engine.py:165-172: Poisson batches, empty ones included
            return DPDataLoader.from_data_loader(
                data_loader, generator=self.secure_rng, distributed=False, batch_first=batch_first,
                rand_on_empty=rand_on_empty,
            )
        if self.secure_mode:
            return switch_generator(data_loader=data_loader, generator=self.secure_rng)
        return data_loader

    def _prepare_model(
        self,
        module: nn.Module,
        *,
        batch_first: bool = True,
        max_grad_norm: Union[float, List[float]] = 1.0,
        loss_reduction: str = "mean",
        grad_sample_mode: str = "hooks",
        wrap_model: bool = True,
    ) -> Union[AbstractGradSampleModule, GradSampleHooks]:
        if wrap_model and isinstance(module, AbstractGradSampleModule):
            if (
                module.batch_first != batch_first
                or module.loss_reduction != loss_reduction
                or type(module) is not get_gsm_class(grad_sample_mode)
            ):
                raise ValueError(
                    f"Pre-existing GradSampleModule doesn't match new arguments."
                    f"Got: module.batch_first: {module.batch_first}, module.loss_reduction: {module.loss_reduction}, type(module): {type(module)}"
                    f"Requested: batch_first:{batch_first}, loss_reduction: {loss_reduction}, grad_sample_mode: {grad_sample_mode} "
                    f"Please pass vanilla nn.Module instead"
                )
            return module
        extra = {"max_grad_norm": max_grad_norm} if grad_sample_mode == "ghost" else {}
        return prepare_module(
            module,
            grad_sample_mode=grad_sample_mode,
            batch_first=batch_first,
            loss_reduction=loss_reduction,
            wrap_model=wrap_model,
            **extra,
        )

    def _prepare_criterion(self, *, module, optimizer, criterion, loss_reduction: str = "mean", **kwargs):
        return DPLossFastGradientClipping(module, optimizer, criterion, loss_reduction)

    # ---- the entry point ----------------------------------------------------------------
    def make_private(
        self,
        *,
        module: nn.Module,
        optimizer: optim.Optimizer,
        criterion=nn.CrossEntropyLoss(),
        data_loader: DataLoader,
        noise_multiplier: float,
        max_grad_norm: Union[float, List[float]],
        batch_first: bool = True,
        loss_reduction: str = "mean",
        poisson_sampling: bool = True,
        clipping: str = "flat",
        noise_generator=None,
        grad_sample_mode: str = "hooks",
        wrap_model: bool = True,
        rand_on_empty: bool = False,
        **kwargs,
    ):
        """Returns ``(module, optimizer, data_loader)``, or with a ghost mode
        ``(module, optimizer, criterion, data_loader)`` (privacy_engine.py:307-475)."""
        if noise_generator and self.secure_mode:
            raise ValueError("Passing seed is prohibited in secure mode")
        model_parameters = set(module.parameters())
        for p in chain.from_iterable(g["params"] for g in optimizer.param_groups):
            if p not in model_parameters:
                raise ValueError("Module parameters are different than optimizer Parameters")
        if isinstance(module, torch.nn.parallel.DistributedDataParallel):
            raise NotImplementedError("data-parallel modules are outside this build (one GPU)")

        module = self._prepare_model(
            module,
            batch_first=batch_first,
            max_grad_norm=max_grad_norm,
            loss_reduction=loss_reduction,
            grad_sample_mode=grad_sample_mode,
            wrap_model=wrap_model,
        )
        if poisson_sampling:
            # a second backward pass before the step would mix two Poisson draws (privacy_engine.py:429-430)
            module.forbid_grad_accumulation()
        data_loader = self._prepare_data_loader(
            data_loader, poisson_sampling=poisson_sampling, batch_first=batch_first, rand_on_empty=rand_on_empty
        )
        sample_rate = 1 / len(data_loader)
        expected_batch_size = int(len(data_loader.dataset) * sample_rate)
        optimizer = self._prepare_optimizer(
            optimizer=optimizer,
            noise_multiplier=noise_multiplier,
            max_grad_norm=max_grad_norm,
            expected_batch_size=expected_batch_size,
            loss_reduction=loss_reduction,
            noise_generator=noise_generator,
            distributed=False,
            clipping=clipping,
            grad_sample_mode=grad_sample_mode,
            **kwargs,
        )
        optimizer.attach_step_hook(self.accountant.get_optimizer_hook_fn(sample_rate=sample_rate))
        if "ghost" in grad_sample_mode:
            criterion = self._prepare_criterion(
                module=module, optimizer=optimizer, criterion=criterion, loss_reduction=loss_reduction, **kwargs
            )
            return module, optimizer, criterion, data_loader
        return module, optimizer, data_loader
