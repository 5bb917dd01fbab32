"""``DPOptimizer`` on the HIP kernels (mirror of opacus/optimizers/optimizer.py).

Same life cycle as the reference: ``step()`` -> ``pre_step()`` -> ``clip_and_accumulate()``
-> ``add_noise()`` -> ``scale_grad()`` -> step hook -> the wrapped optimizer's ``step()``.
What changes is how many times the per-sample gradients cross HBM:

  * per-sample squared norms come for free from the sampler kernels that wrote the
    per-sample gradients (they ride on the tensor); only tensors without a valid one are
    read, all of them in one multi-tensor launch;
  * the clip factor is one tiny kernel;
  * ``sum_n clip[n] * gs[n]`` reads every per-sample gradient exactly once, all parameters
    of a dtype in one launch;
  * noise, the add and the division by the batch size are one kernel over all parameters
    that draws Philox normals in registers, instead of zeros + normal + add + div each.
"""

from __future__ import annotations

import logging
import os
from collections import defaultdict
from typing import Callable, Dict, List, Optional, Tuple, Union

import torch
from torch import nn
from torch.optim import Optimizer

from .. import kernels
from ..grad_sample._common import cached_sumsq
from ..grad_sample.lazy import LazyLinearGradSample
from .utils import params

logger = logging.getLogger(__name__)
logger.disabled = True

# Units of generator offset one noise call consumes (torch wants multiples of 4).
_OFFSET_PER_CALL = 4


def _mark_as_processed(obj: Union[torch.Tensor, List[torch.Tensor]]):
    """Flags gradients as consumed by a step so that using them twice is caught (optimizer.py:32-58)."""
    if isinstance(obj, (torch.Tensor, LazyLinearGradSample)):
        obj._processed = True
    elif isinstance(obj, list):
        for x in obj:
            x._processed = True


def _check_processed_flag_tensor(x: torch.Tensor):
    if "_processed" in getattr(x, "__dict__", ()):
        raise ValueError(
            "Gradients haven't been cleared since the last optimizer step. "
            "In order to obtain privacy guarantees you must call optimizer.zero_grad()"
            "on each step"
        )


def _check_processed_flag(obj: Union[torch.Tensor, List[torch.Tensor]]):
    if isinstance(obj, (torch.Tensor, LazyLinearGradSample)):
        _check_processed_flag_tensor(obj)
    elif isinstance(obj, list):
        for x in obj:
            _check_processed_flag_tensor(x)


# XORed into the torch generator's seed to make the Philox key of the noise kernels. torch's own
# kernels (dropout, randn, initialisers) key Philox with the bare seed and lay offset and thread
# index across the counter differently from the noise kernel, so that with a shared key a
# noise block could coincide with a block some torch kernel draws; a key of its own keeps
# the noise independent of every other use of the generator.
_NOISE_KEY_DOMAIN = 0x44504B5F4E4F4953


def philox_stream(
    generator: Optional[torch.Generator], device: torch.device, calls: int = 1, secure: bool = False
) -> Tuple[int, int]:
    """``(seed, offset)`` for ``calls`` noise kernel launches (each may use up to four
    consecutive offsets), advancing the generator.

    A generator on the GPU (the default one when ``generator`` is None) supplies the key
    (its seed, moved into a domain of its own) and the offset, which moves on, so
    ``torch.manual_seed`` / ``generator.manual_seed`` make runs repeat. A CPU generator
    cannot share an offset with the device; two 62-bit draws from it become the key and
    the offset, which keeps the same determinism.

    ``secure``: key and offset are 126 fresh bits from ``os.urandom`` for every call and
    no generator is consulted, so no seed a user or a library sets can reproduce or predict
    the noise. Philox4x32-10 itself is a counter-based statistical generator, not a
    cryptographic one (the reference's secure mode draws from torchcsprng).
    """
    if secure:
        raw = os.urandom(16)
        return int.from_bytes(raw[:8], "little"), int.from_bytes(raw[8:], "little") >> 2
    if generator is None:
        generator = torch.cuda.default_generators[device.index if device.index is not None else torch.cuda.current_device()]
    if generator.device.type == "cuda":
        seed = generator.initial_seed() ^ _NOISE_KEY_DOMAIN
        offset = generator.get_offset()
        generator.set_offset(offset + _OFFSET_PER_CALL * calls)
        return seed, offset
    draws = torch.randint(0, 2**62, (2,), generator=generator, dtype=torch.int64)
    return int(draws[0]), int(draws[1]) * _OFFSET_PER_CALL


def _generate_noise(std: float, reference: torch.Tensor, generator=None, secure_mode: bool = False) -> torch.Tensor:
    """Gaussian noise of ``reference``'s shape and dtype (optimizer.py:104-169).

    ``std == 0`` gives exact zeros without touching the generator. ``secure_mode`` sums
    four draws and halves, as the reference does against floating-point attacks.
    """
    out = torch.zeros(reference.shape, device=reference.device, dtype=reference.dtype)
    if std == 0:
        return out
    seed, offset = philox_stream(generator, reference.device, secure=secure_mode)
    kernels.add_noise(out, out, std, 1.0, seed, offset, draws=4 if secure_mode else 1)
    return out


class DPOptimizer(Optimizer):
    """Wraps a ``torch.optim.Optimizer``: clips per-sample gradients to ``max_grad_norm``,
    sums them, adds ``N(0, (noise_multiplier * max_grad_norm)^2)`` and rescales
    (optimizer.py:172-581). Per-sample gradients are read from ``p.grad_sample``."""

    def __init__(
        self,
        optimizer: Optimizer,
        *,
        noise_multiplier: float,
        max_grad_norm: float,
        expected_batch_size: Optional[int],
        loss_reduction: str = "mean",
        generator=None,
        secure_mode: bool = False,
        **kwargs,
    ):
        if loss_reduction not in ("mean", "sum"):
            raise ValueError(f"Unexpected value for loss_reduction: {loss_reduction}")
        if loss_reduction == "mean" and expected_batch_size is None:
            raise ValueError("You must provide expected batch size of the loss reduction is mean")
        self.original_optimizer = optimizer
        self.noise_multiplier = noise_multiplier
        self.max_grad_norm = max_grad_norm
        self.loss_reduction = loss_reduction
        self.expected_batch_size = expected_batch_size
        self.step_hook = None
        self.generator = generator
        self.secure_mode = secure_mode
        self._step_skip_queue = []
        self._is_last_step_skipped = False
        for p in self.params:
            p.summed_grad = None

    # ---- per-sample gradient access -----------------------------------------------------
    def _get_flat_grad_sample(self, p: torch.Tensor, factors_ok: bool = False):
        """``p.grad_sample`` as one tensor; a list from several backward passes is
        concatenated along the batch (optimizer.py:252-292). A Linear weight's gradient that is
        still held as its two factors (``lazy_linear_grad_sample``) is returned as it is to a caller
        that says it can work from them, and formed for any other."""
        if not hasattr(p, "grad_sample"):
            raise ValueError("Per sample gradient not found. Are you using GradSampleModule?")
        if p.grad_sample is None:
            raise ValueError("Per sample gradient is not initialized. Not updated in backward pass?")
        if isinstance(p.grad_sample, torch.Tensor):
            return p.grad_sample
        if isinstance(p.grad_sample, LazyLinearGradSample):
            return p.grad_sample if factors_ok else p.grad_sample.materialize()
        if isinstance(p.grad_sample, list):
            return torch.cat(p.grad_sample, dim=0)
        raise ValueError(f"Unexpected grad_sample type: {type(p.grad_sample)}")

    def signal_skip_step(self, do_skip=True):
        """Queues whether the next ``step`` only clips and accumulates (virtual batches,
        optimizer.py:294-329)."""
        self._step_skip_queue.append(do_skip)

    def _check_skip_next_step(self, pop_next=True):
        if self._step_skip_queue:
            return self._step_skip_queue.pop(0) if pop_next else self._step_skip_queue[0]
        return False

    @property
    def params(self) -> List[nn.Parameter]:
        return params(self)

    @property
    def grad_samples(self) -> List[torch.Tensor]:
        return [self._get_flat_grad_sample(p) for p in self.params]

    @property
    def accumulated_iterations(self) -> int:
        """Backward passes accumulated in ``grad_sample`` (1 for a tensor, the length of a
        list); must agree across parameters (optimizer.py:348-376)."""
        vals = set()
        for p in self.params:
            if not hasattr(p, "grad_sample"):
                raise ValueError("Per sample gradient not found. Are you using GradSampleModule?")
            if isinstance(p.grad_sample, (torch.Tensor, LazyLinearGradSample)):
                vals.add(1)
            elif isinstance(p.grad_sample, list):
                vals.add(len(p.grad_sample))
            else:
                raise ValueError(f"Unexpected grad_sample type: {type(p.grad_sample)}")
        if len(vals) > 1:
            raise ValueError("Number of accumulated steps is inconsistent across parameters")
        return vals.pop()

    # ---- delegation to the wrapped optimizer ------------------------------------------------
    @property
    def param_groups(self) -> List[dict]:
        return self.original_optimizer.param_groups

    @param_groups.setter
    def param_groups(self, param_groups: List[dict]):
        self.original_optimizer.param_groups = param_groups

    @property
    def state(self) -> defaultdict:
        return self.original_optimizer.state

    @state.setter
    def state(self, state: defaultdict):
        self.original_optimizer.state = state

    @property
    def defaults(self) -> dict:
        return self.original_optimizer.defaults

    @defaults.setter
    def defaults(self, defaults: dict):
        self.original_optimizer.defaults = defaults

    def attach_step_hook(self, fn: Callable[["DPOptimizer"], None]):
        """``fn(optimizer)`` runs after noise and scaling, before the wrapped step (privacy accounting)."""
        self.step_hook = fn

    # ---- the hot path ---------------------------------------------------------------------
    def _per_param_sumsq(self, plist: List[nn.Parameter], flats: List[torch.Tensor]) -> torch.Tensor:
        """``[K, n]`` squared norms: cached ones from the sampler kernels where they are still
        valid, one multi-tensor pass over the rest."""
        n = flats[0].shape[0]
        dev = flats[0].device
        rows: List[Optional[torch.Tensor]] = []
        missing: Dict[Tuple[torch.dtype, torch.device], List[int]] = {}
        for k, (p, g) in enumerate(zip(plist, flats)):
            if isinstance(g, LazyLinearGradSample):
                ss = g.sumsq  # closed form or Gram contraction of the factors
            else:
                ss = cached_sumsq(p.grad_sample) if isinstance(p.grad_sample, torch.Tensor) else None
            rows.append(ss)
            if ss is None:
                missing.setdefault((g.dtype, g.device), []).append(k)
        for (_, _), idxs in missing.items():
            got = kernels.sumsq_rows([flats[k] for k in idxs])
            for j, k in enumerate(idxs):
                rows[k] = got[j]
        return torch.stack([r.to(dev) for r in rows], dim=0) if len(rows) > 1 else rows[0].to(dev).reshape(1, n)

    def _clip_factors(self, plist: List[nn.Parameter], flats: List[torch.Tensor]) -> torch.Tensor:
        """Per-sample clip factors ``min(1, C / (norm + 1e-6))`` of the whole gradient
        (optimizer.py:444-455): ``float32[n]``. Subclasses with another clipping rule return
        their own vector, or a ``[K, n]`` table with a row per parameter."""
        n = len(flats[0])
        if n == 0:
            return torch.zeros((0,), device=flats[0].device, dtype=torch.float32)
        sumsq = self._per_param_sumsq(plist, flats)
        return kernels.clip_factor(sumsq, float(self.max_grad_norm))[1]

    def clip_and_accumulate(self):
        """Clips every sample's gradient to ``max_grad_norm`` and adds the clipped gradients
        into ``p.summed_grad`` (optimizer.py:432-475)."""
        plist = self.params
        flats = []
        for p in plist:
            _check_processed_flag(p.grad_sample)
            g = self._get_flat_grad_sample(p, factors_ok=True)
            if not kernels.supported_dtype(g.dtype):
                raise TypeError(f"per-sample gradients must be float32 or bfloat16 on this path, got {g.dtype}")
            flats.append(g)
        clip = self._clip_factors(plist, flats)
        per_layer = clip.dim() == 2
        # one launch per (device, per-sample dtype, parameter dtype, fresh/accumulate) group
        groups: Dict[tuple, List[int]] = {}
        for k, (p, g) in enumerate(zip(plist, flats)):
            out_dtype = p.dtype if kernels.supported_dtype(p.dtype) else torch.float32
            if isinstance(g, LazyLinearGradSample):
                # a Linear weight held as activations and backprops: its clipped sum is one
                # contraction over samples and positions with the clip factors as coefficients
                total = g.weighted_sum((clip[k] if per_layer else clip).to(g.device), out_dtype=out_dtype)
                if p.summed_grad is None:
                    p.summed_grad = total
                else:
                    p.summed_grad += total
                continue
            if p.summed_grad is None:
                p.summed_grad = torch.empty(g.shape[1:], device=g.device, dtype=out_dtype)
                fresh = True
            else:
                fresh = False
                if not p.summed_grad.is_contiguous() or p.summed_grad.dtype != out_dtype:
                    raise ValueError("summed_grad must be a dense tensor of the parameter's dtype")
            groups.setdefault((g.device, g.dtype, out_dtype, fresh), []).append(k)
        for (dev, _, _, fresh), idxs in groups.items():
            factors = clip[idxs] if per_layer and len(idxs) != len(plist) else clip
            kernels.clip_accumulate(
                [flats[k] for k in idxs], factors.to(dev), [plist[k].summed_grad for k in idxs], accumulate=not fresh
            )
        for p in plist:
            if p.summed_grad.dtype != p.dtype:
                p.summed_grad = p.summed_grad.to(p.dtype)
            _mark_as_processed(p.grad_sample)

    def _noise_std(self) -> float:
        return self.noise_multiplier * self.max_grad_norm

    def _add_noise_scaled(self, denom: float):
        std = self._noise_std()
        draws = 4 if self.secure_mode else 1
        # one launch per (device, dtype) group of parameters, all drawing from one stream
        groups: Dict[tuple, Tuple[list, list]] = {}
        for p in self.params:
            _check_processed_flag(p.summed_grad)
            summed = p.summed_grad
            if not kernels.supported_dtype(summed.dtype):
                raise TypeError(f"summed_grad must be float32 or bfloat16 on this path, got {summed.dtype}")
            if not summed.is_contiguous():
                summed = summed.contiguous()
            if summed.numel() == 0:
                p.grad = torch.empty(p.shape, device=summed.device, dtype=summed.dtype)
                _mark_as_processed(p.summed_grad)
                continue
            grad = torch.empty(p.shape, device=summed.device, dtype=summed.dtype)
            ss, gg = groups.setdefault((summed.device, summed.dtype), ([], []))
            ss.append(summed)
            gg.append(grad)
            p.grad = grad
            _mark_as_processed(p.summed_grad)
        for (dev, _), (ss, gg) in groups.items():
            launches = -(-len(ss) // kernels.DPK_MULTI_MAX)
            if std == 0:
                seed = offset = 0  # nothing is drawn and the generator stays where it is
            else:
                seed, offset = philox_stream(self.generator, dev, calls=launches, secure=self.secure_mode)
            kernels.add_noise_multi(ss, gg, std, denom, seed, offset, draws=draws)

    def add_noise(self):
        """``p.grad = (p.summed_grad + N(0, std^2)).view_as(p)`` (optimizer.py:477-493)."""
        self._add_noise_scaled(1.0)

    def scale_grad(self):
        """Divides ``p.grad`` by ``expected_batch_size * accumulated_iterations`` for a
        mean-reduced loss; nothing for a sum (optimizer.py:495-504)."""
        if self.loss_reduction == "mean":
            denom = float(self.expected_batch_size * self.accumulated_iterations)
            for p in self.params:
                g = p.grad
                if g.is_cuda and g.is_contiguous() and kernels.supported_dtype(g.dtype):
                    kernels.add_noise(g, g, 0.0, denom, 0, 0)
                else:
                    p.grad /= denom

    def _noise_and_scale(self):
        """``add_noise`` then ``scale_grad``; one kernel when neither method has been
        overridden by a subclass."""
        cls = type(self)
        fused = cls.add_noise is DPOptimizer.add_noise and cls.scale_grad is DPOptimizer.scale_grad
        if fused:
            denom = 1.0
            if self.loss_reduction == "mean":
                denom = float(self.expected_batch_size * self.accumulated_iterations)
            self._add_noise_scaled(denom)
        else:
            self.add_noise()
            self.scale_grad()

    # ---- the whole step of a small model as one launch ----------------------------------------
    FUSED_STEP_MAX_ELEMENTS = 1 << 20  # columns (in units of 4 where all tensors allow it) up to which it is used

    def _fused_small_step(self) -> bool:
        """clip_and_accumulate + add_noise + scale_grad as one kernel launch, when nothing about this
        step needs them apart: flat clipping by this class's own rule, no virtual step pending or
        behind, one device and dtype, per-sample gradients that still carry the squared norms their
        samplers left, 64 to 1024 samples and few enough columns that the sum runs in its
        small-tensor shape. ``p.grad`` and ``p.summed_grad`` hold the bits the three methods leave
        (same kernels' arithmetic in the same order, same noise stream); they are views of two flat
        buffers, one allocation each instead of one per parameter. Returns False when the step has
        to take the separate methods."""
        cls = type(self)
        if (
            cls.clip_and_accumulate is not DPOptimizer.clip_and_accumulate
            or cls._clip_factors is not DPOptimizer._clip_factors
            or cls.add_noise is not DPOptimizer.add_noise
            or cls.scale_grad is not DPOptimizer.scale_grad
            or self._check_skip_next_step(pop_next=False)
        ):
            return False
        plist = self.params
        if not plist or len(plist) > kernels.DPK_MULTI_MAX:
            return False
        flats, sumsqs = [], []
        first = plist[0].grad_sample if hasattr(plist[0], "grad_sample") else None
        if not isinstance(first, torch.Tensor) or not first.is_cuda:
            return False
        n, dev, gdt, odt = first.shape[0], first.device, first.dtype, plist[0].dtype
        if not (kernels.CLIP_NOISE_STEP_MIN_N <= n <= kernels.CLIP_NOISE_STEP_MAX_N):
            return False
        if not (kernels.native_dtype(gdt) and kernels.native_dtype(odt)):
            return False
        total, vec = 0, True
        for p in plist:
            g = getattr(p, "grad_sample", None)
            if (
                not isinstance(g, torch.Tensor) or p.summed_grad is not None or hasattr(g, "_processed")
                or g.device != dev or g.dtype != gdt or p.dtype != odt or g.shape[0] != n or not g.is_contiguous()
                or g.numel() == 0
            ):
                return False
            ss = cached_sumsq(g)
            if ss is None or ss.device != dev:
                return False
            flats.append(g)
            sumsqs.append(ss)
            P = g.numel() // n
            total += P
            vec = vec and P % 4 == 0
        if total // (4 if vec else 1) >= min(self.FUSED_STEP_MAX_ELEMENTS, 256 * 1024):
            return False  # the separate kernels stream tensors of this size
        # one buffer for the sums and one for the gradients, every parameter's piece at a multiple of 16 bytes
        offs, at = [], 0
        for g in flats:
            offs.append(at)
            at += -(-(g.numel() // n) // 8) * 8
        flat_sum = torch.empty(at, device=dev, dtype=odt)
        flat_grad = torch.empty(at, device=dev, dtype=odt)
        summed = [flat_sum[o : o + g.numel() // n] for o, g in zip(offs, flats)]
        grads = [flat_grad[o : o + g.numel() // n] for o, g in zip(offs, flats)]
        if self._step_skip_queue:
            self._step_skip_queue.pop(0)  # (False: checked above) this step's entry of the queue
        std = self._noise_std()
        denom = 1.0
        if self.loss_reduction == "mean":
            denom = float(self.expected_batch_size * self.accumulated_iterations)
        if std == 0:
            seed = offset = 0  # nothing is drawn and the generator stays where it is
        else:
            seed, offset = philox_stream(self.generator, dev, calls=1, secure=self.secure_mode)
        kernels.clip_noise_step(
            flats, sumsqs, grads, summed, float(self.max_grad_norm), std, denom, seed, offset, draws=4 if self.secure_mode else 1
        )
        for p, g, sm, gr in zip(plist, flats, summed, grads):
            p.summed_grad = sm.view(p.shape)
            p.grad = gr.view(p.shape)
            _mark_as_processed(g)
            _mark_as_processed(p.summed_grad)
        return True

    def zero_grad(self, set_to_none: bool = False):
        """Clears ``p.grad``, ``p.grad_sample`` and, unless the last step was a skipped
        (virtual) one, ``p.summed_grad`` (optimizer.py:506-537)."""
        for p in self.params:
            p.grad_sample = None
            if not self._is_last_step_skipped:
                p.summed_grad = None
        self.original_optimizer.zero_grad(set_to_none)

    def pre_step(self, closure: Optional[Callable[[], float]] = None) -> Optional[float]:
        """Everything before the wrapped optimizer's step; returns False when this step is
        a skipped one that only accumulated (optimizer.py:539-563)."""
        if len(self.params) == 0:
            return True
        if not self._fused_small_step():
            self.clip_and_accumulate()
            if self._check_skip_next_step():
                self._is_last_step_skipped = True
                return False
            self._noise_and_scale()
        if self.step_hook:
            self.step_hook(self)
        self._is_last_step_skipped = False
        return True

    def step(self, closure: Optional[Callable[[], float]] = None) -> Optional[float]:
        if closure is not None:
            with torch.enable_grad():
                closure()
        if self.pre_step():
            return self.original_optimizer.step()
        return None

    def __repr__(self):
        return self.original_optimizer.__repr__()

    def state_dict(self):
        return self.original_optimizer.state_dict()

    def load_state_dict(self, state_dict) -> None:
        self.original_optimizer.load_state_dict(state_dict)
