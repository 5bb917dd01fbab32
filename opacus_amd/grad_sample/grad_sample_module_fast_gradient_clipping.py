"""Ghost clipping / fast gradient clipping hooks.

Mirror of opacus/grad_sample/grad_sample_module_fast_gradient_clipping.py: on the first
backward pass every parameter receives a per-sample gradient NORM (``p._norm_sample``)
instead of a per-sample gradient. Layers with a registered norm sampler (Linear,
Embedding) get it from the ghost-norm kernels without the gradient ever existing; other
layers have their per-sample gradient formed by the grad sampler, reduced to a norm and
dropped at once. ``get_clipping_coef`` then yields ``min(1, C / (norm + 1e-6))``.

One kind of parameter tying is taken under ghost clipping, which the reference refuses
altogether (:172-179): an ``nn.Embedding`` whose table is also the weight of an ``nn.Linear``
(tied input and output embeddings). The norm of the sum of the two layers' gradients is
their two ghost norms plus twice a cross term, ``kernels.tied_embedding_cross_term``.

``single_backward=True`` (the default) replaces the second backward pass: the hooks keep every
layer's (activations, backprops) of the first pass, and once the clipping coefficients are known the
clipped gradient sum of each layer is formed from them directly: one contraction over samples
and positions with the coefficients applied inside the kernel for a Linear layer
(``kernels.linear_weighted_sum[_multi]``, ``linear_bias_weighted_sum``), the per-id sum of the
weighted backprop rows for an Embedding (``kernels.embedding_weighted_sum``), the layer's grad
sampler and the clip-weighted sum for anything else. The sum is the one the
second pass would have left in ``p.grad`` (the gradient of ``sum_n coef[n] loss[n]`` is linear
in the per-sample backprops); what is saved is the pass's walk back through the activations,
at the price of keeping the backprops alive until the coefficients exist (the first pass no
longer retains the graph, so the peak is about that of the reference's retained graph).
``single_backward=False`` runs the reference's two passes (fast_gradient_clipping_utils.py:179-201).
Only autograd's second pass sees a dependence of the loss on trainable parameters other than
through the hooked layers (a regulariser on the weights, ``F.linear(x, layer.weight)`` beside the
layer's own call). ``single_pass_is_exact`` therefore walks the loss's graph before every first
pass and compares, parameter by parameter, the uses autograd has recorded with the uses the
forward hooks have seen; a step whose graph holds any other use runs the reference's two passes
(with one warning), so the default never drops a gradient term.

Norm samples are kept in float32 whatever the dtype of the backprops (the kernels
accumulate in fp32; rounding a norm to bf16 before it meets the other parameters' norms
would only lose bits).
"""

from __future__ import annotations

import logging
from typing import List

import torch
import torch.nn as nn

from .. import kernels
from ..utils.module_utils import requires_grad, trainable_modules, trainable_parameters
from ._common import cached_sumsq
from .grad_sample_module import (
    GradSampleHooks,
    call_sampler,
    create_or_accumulate_grad_sample,
    promote_current_grad_sample,
)
from .gsm_base import AbstractGradSampleModule

logger = logging.getLogger(__name__)
logger.disabled = True


def create_norm_sample(*, param: torch.Tensor, grad_sample: torch.Tensor, max_batch_len: int) -> None:
    """``param._norm_sample`` = per-sample 2-norm of ``grad_sample``; an empty tensor for an
    empty batch (grad_sample_module_fast_gradient_clipping.py:42-70)."""
    if not param.requires_grad:
        return
    if max_batch_len == 0:
        param._norm_sample = torch.zeros((0,), device=grad_sample.device, dtype=torch.float32)
        return
    ss = cached_sumsq(grad_sample)
    if ss is None:
        ss = kernels.sumsq_rows([grad_sample])[0]
    param._norm_sample, _ = kernels.clip_factor(ss.reshape(1, -1), 1.0)


class GradSampleHooksFastGradientClipping(GradSampleHooks):
    """Hooks object computing per-sample gradient norms (ghost clipping where a norm
    sampler exists, fast gradient clipping elsewhere)."""

    NORM_SAMPLERS = {}
    CAN_SKIP_AUTOGRAD_WEIGHT_GRADS = False  # the second backward pass is autograd's
    KEEP_GRAD_SAMPLES_BELOW = 1 << 22  # elements per layer and pass, single_backward only

    def __init__(
        self,
        m: nn.Module,
        *,
        batch_first=True,
        loss_reduction="mean",
        strict: bool = True,
        force_functorch=False,
        max_grad_norm=1,
        use_ghost_clipping=True,
        single_backward: bool = True,
    ):
        super().__init__(
            m, batch_first=batch_first, loss_reduction=loss_reduction, strict=strict, force_functorch=force_functorch
        )
        self.single_backward = single_backward
        self._kept_passes = []
        self._pending_ghost = []
        self.trainable_parameters = [p for _, p in trainable_parameters(self._module)]
        self._tied_embedding_weights = self._find_tied_embedding_weights()

        self.max_grad_norm = max_grad_norm
        self.use_ghost_clipping = use_ghost_clipping
        self._per_sample_gradient_norms = None

    # ---- tied input / output embeddings ------------------------------------------------
    def _find_tied_embedding_weights(self) -> set:
        """ids of the weights owned by exactly one ``nn.Embedding`` and one ``nn.Linear``."""
        owners = {}
        for _, m in trainable_modules(self._module):
            for name, p in m.named_parameters(recurse=False):
                owners.setdefault(id(p), []).append((m, name))
        tied = set()
        for pid, uses in owners.items():
            if (
                len(uses) == 2
                and {type(m) for m, _ in uses} == {nn.Embedding, nn.Linear}
                and all(name == "weight" for _, name in uses)
            ):
                tied.add(pid)
        return tied

    def _tied_embedding_norm(self, param, module, activations, backprops, scale, ns):
        """Keeps this layer's share of a tied table; once both layers of the pass have
        reported, returns ``sqrt(|G_emb|^2 + |G_head|^2 + 2 <G_emb, G_head>)``. Until then the
        layer's own norm stands in."""
        parts = param.__dict__.setdefault("_tied_parts", {})
        parts["emb" if isinstance(module, nn.Embedding) else "head"] = (activations[0], backprops, scale, ns)
        if len(parts) < 2:
            return ns
        del param.__dict__["_tied_parts"]
        ids, e, s_e, ns_e = parts["emb"]
        a, g, s_h, ns_h = parts["head"]
        cross = kernels.tied_embedding_cross_term(ids, e, a, g, scale=s_e * s_h)
        return (ns_e.float().square() + ns_h.float().square() + 2.0 * cross).clamp_(min=0).sqrt_()

    def add_hooks(self, *, loss_reduction: str = "mean", batch_first: bool = True, force_functorch: bool = False) -> None:
        super().add_hooks(loss_reduction=loss_reduction, batch_first=batch_first, force_functorch=force_functorch)
        self._first_pass_leaves = {}
        self._first_pass_open = False
        self.autograd_grad_sample_hooks.append(
            self._module.register_forward_pre_hook(self._note_model_inputs, with_kwargs=True)
        )

    # ---- what the first backward pass has to reach -----------------------------------------
    def _note_first_pass_leaves(self, module: nn.Module, forward_input, forward_output) -> None:
        """The norm pass needs the gradient of every hooked module's OUTPUT, never a weight
        gradient (``optimizer.zero_grad()`` discards those right after,
        fast_gradient_clipping_utils.py:190-191). Autograd computes exactly the output
        gradients, and skips every weight-gradient GEMM, when it is asked only for the
        tensors at the start of the graph: the outputs of modules none of whose inputs
        requires grad (or, where such an output is not a single tensor, their parameters),
        and inputs that are leaves requiring grad."""
        tensors = [t for t in forward_input if isinstance(t, torch.Tensor)]
        if not any(t.requires_grad for t in tensors):
            if isinstance(forward_output, torch.Tensor) and forward_output.requires_grad:
                # kept with its version: an in-place op on it later moves the tensor to
                # another node of the graph, and the module's parameters are asked for instead
                self._first_pass_leaves[id(forward_output)] = (forward_output, forward_output._version, module)
            else:
                for _, p in trainable_parameters(module):
                    self._first_pass_leaves[id(p)] = (p, None, module)
        for t in tensors:
            if t.requires_grad and t.is_leaf:
                self._first_pass_leaves[id(t)] = (t, None, module)

    def _note_model_inputs(self, _module, args, kwargs) -> None:
        """Inputs of the model that carry a graph of their own: a leaf that requires grad is
        one more leaf to reach; a computed tensor that requires grad has leaves this object
        cannot see, and the first pass then stays unrestricted."""
        # records are made by backward hooks and consumed at the end of the same backward();
        # anything still here was left by one that did not get that far
        self._kept_passes = []
        self._pending_ghost = []
        stack = list(args) + list(kwargs.values())
        while stack:
            t = stack.pop()
            if isinstance(t, (list, tuple)):
                stack.extend(t)
            elif isinstance(t, dict):
                stack.extend(t.values())
            elif isinstance(t, torch.Tensor) and t.requires_grad:
                if t.is_leaf:
                    self._first_pass_leaves[id(t)] = (t, None, None)
                else:
                    self._first_pass_open = True

    def first_backward_inputs(self) -> List[torch.Tensor]:
        """Leaves to pass as ``inputs=`` to the first backward pass of ghost clipping (empty:
        do not restrict the pass); the record starts afresh for the next forward pass."""
        leaves = []
        if not self._first_pass_open:
            for t, version, module in self._first_pass_leaves.values():
                if version is None or t._version == version:
                    leaves.append(t)
                else:
                    leaves.extend(p for _, p in trainable_parameters(module))
        self._first_pass_leaves = {}
        self._first_pass_open = False
        return leaves

    # ---- is the clipped sum of the hooked layers the whole gradient? ------------------------
    def single_pass_is_exact(self, root: torch.Tensor) -> bool:
        """True when every use of a trainable parameter in the graph of ``root`` (the reduced
        loss) is one that a forward hook has seen, i.e. when the clipped sums formed from the
        hooked layers' (activations, backprops) are all that the reference's second pass would
        leave in ``p.grad`` (fast_gradient_clipping_utils.py:193-201).

        Autograd keeps one accumulation node per leaf, with one incoming edge per use of the leaf.
        A hooked layer's call uses each of its own parameters once, and the forward hooks count
        the calls in ``p._forward_counter``. More edges than calls (a regulariser on the weights,
        a functional use beside the layer's own), or a trainable leaf that no hooked layer owns,
        means a term that only a second pass would differentiate. A layer that uses a parameter
        several times per call is reported as inexact too, which costs that model the second pass
        and nothing else."""
        fn = root.grad_fn
        if fn is None:
            return True
        own = {id(p): p for p in self.trainable_parameters}
        uses = {}
        seen = {fn}
        stack = [fn]
        while stack:
            node = stack.pop()
            for nxt, _ in node.next_functions:
                if nxt is None:
                    continue
                var = getattr(nxt, "variable", None)
                if var is not None:  # an accumulation node: one edge = one use of the leaf
                    if var.requires_grad:
                        uses[id(var)] = uses.get(id(var), 0) + 1
                        if id(var) not in own and isinstance(var, nn.Parameter):
                            return False  # a trainable parameter outside the wrapped module's hooked layers
                elif nxt not in seen:
                    seen.add(nxt)
                    stack.append(nxt)
        for pid, count in uses.items():
            p = own.get(pid)
            if p is not None and count > getattr(p, "_forward_counter", 0):
                return False
        return True

    # ---- Linear ghost norms of a whole pass in one launch ----------------------------------
    def _defer_linear_ghost_norm(self, module: nn.Module, activations, backprops: torch.Tensor, scale: float):
        """With ``single_backward`` the (activations, backprops) of every layer stay alive until
        the coefficients exist anyway, so the Linear layers' norms need not be formed hook by
        hook: the hook hands out the tensors that will hold them and queues the layer;
        ``flush_ghost_norms`` forms them all in one pooled launch (the tile pairs of all layers
        fill the device together, kernels.linear_ghost_norm_multi). Returns None when the layer
        is not queued (another sampler is registered for it, an empty batch, dtypes the kernels
        do not take)."""
        from .linear import compute_linear_norm_sample

        if (
            not self.single_backward
            or self.NORM_SAMPLERS.get(type(module)) is not compute_linear_norm_sample
            or backprops.shape[0] == 0
            or not backprops.is_cuda
            or not kernels.native_dtype(backprops.dtype)  # float16 goes through call_sampler, widened
        ):
            return None
        n, dev = backprops.shape[0], backprops.device
        want_w = module.weight.requires_grad
        want_b = module.bias is not None and module.bias.requires_grad
        nw = torch.empty((n,), dtype=torch.float32, device=dev) if want_w else None
        nb = torch.empty((n,), dtype=torch.float32, device=dev) if want_b else None
        if not self._pending_ghost:
            # runs when the backward pass in flight has finished: the norms are in place by the
            # time backward() returns, whoever reads p._norm_sample next
            torch.autograd.Variable._execution_engine.queue_callback(self.flush_ghost_norms)
        self._pending_ghost.append((backprops, activations[0], scale, nw, nb))
        ret = {}
        if want_w:
            ret[module.weight] = nw
        if want_b:
            ret[module.bias] = nb
        return ret

    def flush_ghost_norms(self) -> None:
        """Forms the queued Linear ghost norms (in place, in the tensors already handed out)."""
        pending, self._pending_ghost = self._pending_ghost, []
        groups = {}
        for item in pending:
            bp = item[0]
            groups.setdefault((bp.shape[0], bp.dtype, bp.device), []).append(item)
        for items in groups.values():
            kernels.linear_ghost_norm_multi(items)

    # ---- clipping coefficient ----------------------------------------------------------
    def get_norm_sample(self) -> torch.Tensor:
        """Per-sample norm over all parameters: 2-norm of the stacked per-parameter norms
        (grad_sample_module_fast_gradient_clipping.py:142-150)."""
        norm, _ = self._norm_and_coef()
        return norm

    def get_clipping_coef(self) -> torch.Tensor:
        """``min(1, C / (norm + 1e-6))`` per sample (:137-140)."""
        _, coef = self._norm_and_coef()
        return coef

    def _norm_and_coef(self):
        self.flush_ghost_norms()
        norm_samples = [p._norm_sample for p in self.trainable_parameters]
        if not norm_samples:
            raise ValueError("no trainable parameter carries a norm sample")
        dev = norm_samples[0].device
        stacked = torch.stack([ns.to(device=dev, dtype=torch.float32).reshape(-1) for ns in norm_samples], dim=0)
        norm, coef = kernels.clip_factor(stacked, float(self.max_grad_norm), is_norm=True)
        self.per_sample_gradient_norms = norm
        return norm, coef

    # ---- hooks ------------------------------------------------------------------------------
    def capture_activations_hook(self, module: nn.Module, forward_input: List[torch.Tensor], _forward_output):
        if (
            not requires_grad(module)
            or not module.training
            or not torch.is_grad_enabled()
            or not self.hooks_enabled
        ):
            return
        if not hasattr(module, "activations"):
            module.activations = []
        # non-tensor inputs (an omitted optional argument passed as None) are not activations
        module.activations.append([t.detach() for t in forward_input if isinstance(t, torch.Tensor)])
        self._note_first_pass_leaves(module, forward_input, _forward_output)
        for _, p in trainable_parameters(module):
            p._forward_counter += 1
            if p._forward_counter == 1:
                p.__dict__.pop("_tied_parts", None)  # left by a backward pass that did not finish
                module.__dict__.pop("_dpk_materialise", None)
            if (
                self.use_ghost_clipping
                and p._forward_counter > 1
                and type(module) in self.NORM_SAMPLERS
                and not getattr(module, "stack_uses", False)  # its uses are contracted together
                and not (id(p) in self._tied_embedding_weights and p._forward_counter == 2)
            ):
                if getattr(self.NORM_SAMPLERS[type(module)], "reference_materialises", False):
                    # a layer type the reference serves by forming the per-sample gradients anyway
                    # (no norm sampler there): used more than once in a pass, it is served that way here too
                    module._dpk_materialise = True
                else:
                    # the norm of a sum of two layers' gradients is not a function of their norms
                    raise NotImplementedError("Parameter tying is not supported with Ghost Clipping")

    def capture_backprops_hook(
        self, module: nn.Module, _forward_input, forward_output, loss_reduction: str, batch_first: bool
    ):
        """Fills ``p._norm_sample`` for the parameters of ``module`` (:181-253)."""
        if not self.hooks_enabled:
            return
        backprops = forward_output[0].detach()
        activations, backprops, scale = self._take_activations(
            module=module, backprops=backprops, loss_reduction=loss_reduction, batch_first=batch_first
        )
        if getattr(module, "stack_uses", False):
            stacked = self._stack_uses(module, activations, backprops)
            if stacked is None:
                return
            activations, backprops = stacked
            for _, p in trainable_parameters(module):
                p._forward_counter += 1  # taken off again below, as for a module used once
        ghost = (
            self.use_ghost_clipping
            and type(module) in self.NORM_SAMPLERS
            and not getattr(module, "_dpk_materialise", False)
        )
        if self.single_backward and ghost:
            self._kept_passes.append((module, activations, backprops, scale, None))
        if ghost:
            norm_samples = self._defer_linear_ghost_norm(module, activations, backprops, scale)
            if norm_samples is None:
                norm_samples = call_sampler(self.NORM_SAMPLERS[type(module)], module, activations, backprops, scale)
            for param, ns in norm_samples.items():
                if param.requires_grad:
                    if id(param) in self._tied_embedding_weights:
                        self.flush_ghost_norms()  # the cross term is combined with finished norms
                        ns = self._tied_embedding_norm(param, module, activations, backprops, scale, ns)
                    param._norm_sample = ns
                    param._forward_counter -= 1
        else:
            sampler = self._sampler_for(module)
            grad_samples = call_sampler(sampler, module, activations, backprops, scale)
            if self.single_backward:
                # small per-sample gradients (norm layers, biases) are kept as they are; large
                # ones are formed again when the coefficients exist
                small = sum(gs.numel() for gs in grad_samples.values()) <= self.KEEP_GRAD_SAMPLES_BELOW
                # (copies: a tensor adopted as p._current_grad_sample has later uses of the module added into it)
                kept_gs = {p: gs.clone() for p, gs in grad_samples.items()} if small else None
                self._kept_passes.append((module, activations, backprops, scale, kept_gs))
            adopt = getattr(sampler, "owns_output", False)
            for param, gs in grad_samples.items():
                create_or_accumulate_grad_sample(
                    param=param, grad_sample=gs, max_batch_len=module.max_batch_len, adopt=adopt
                )
            del grad_samples
            for _, p in trainable_parameters(module):
                p._forward_counter -= 1
                if p._forward_counter == 0:
                    promote_current_grad_sample(p)
                    create_norm_sample(param=p, grad_sample=p.grad_sample, max_batch_len=module.max_batch_len)
                    p.grad_sample = None
        if len(module.activations) == 0 and hasattr(module, "max_batch_len"):
            del module.max_batch_len

    # ---- the clipped sum without a second backward pass ---------------------------------------
    def accumulate_clipped_gradients(self, coef: torch.Tensor) -> None:
        """Adds ``sum_n coef[n] * grad_n`` of every layer seen by the last backward pass to
        ``p.grad``, from the kept (activations, backprops): what the second backward pass of
        ``sum_n coef[n] * loss[n]`` leaves there (fast_gradient_clipping_utils.py:193-201)."""
        from .linear import compute_linear_grad_sample as linear_grad_sampler  # imports this module's package

        kept, self._kept_passes = self._kept_passes, []
        sums = {}

        def add(param, value):
            if not param.requires_grad:
                return
            value = value.reshape(param.shape)
            if id(param) in sums:
                sums[id(param)][1].add_(value.to(sums[id(param)][1].dtype))
            else:
                sums[id(param)] = (param, value)

        # bf16 Linear layers on sequences: the coefficients go onto the accumulators of one
        # contraction over all samples and positions (neither operand is weighted or copied
        # beforehand), and the tiles of all such layers are one pooled launch
        pooled, rest = [], []
        for entry in kept:
            module, activations, backprops = entry[0], entry[1], entry[2]
            if backprops.shape[0] and self._sampler_for(module) is linear_grad_sampler:
                a = activations[0].to(backprops.dtype)
                if module.weight.requires_grad and kernels.linear_weighted_sum_takes(backprops, a):
                    pooled.append((module, a, backprops, entry[3]))
                    continue
            rest.append(entry)
        by_device = {}
        for item in pooled:
            by_device.setdefault(item[2].device, []).append(item)
        for dev, items in by_device.items():
            c = coef.to(device=dev, dtype=torch.float32)
            sums_w = kernels.linear_weighted_sum_multi([(b, a, c, scale) for _, a, b, scale in items])
            for (module, a, backprops, scale), total in zip(items, sums_w):
                add(module.weight, total)
                if module.bias is not None and module.bias.requires_grad:
                    add(module.bias, kernels.linear_bias_weighted_sum(backprops, c, scale=scale))
        del pooled, by_device
        for module, activations, backprops, scale, grad_samples in rest:
            n = backprops.shape[0]
            c = coef.to(device=backprops.device, dtype=torch.float32)
            if n == 0:
                continue
            if self._sampler_for(module) is linear_grad_sampler and kernels.native_dtype(backprops.dtype) and backprops.is_cuda:
                # nn.Linear itself and RNNLinear (not a subclass with a forward of its own) in the shapes and
                # dtypes the pooled contraction does not take: fp32, positions that are not whole k tiles,
                # odd feature sizes. One contraction over all rows with the rows of the backprops weighted
                # on their way into the kernel's LDS tiles: no weighted copy, no library GEMM.
                if module.weight.requires_grad:
                    add(module.weight, kernels.linear_weighted_sum(backprops, activations[0], c, scale=scale))
                if module.bias is not None and module.bias.requires_grad:
                    add(module.bias, kernels.linear_bias_weighted_sum(backprops, c, scale=scale))
            elif self._sampler_for(module) is linear_grad_sampler:  # float16: widened operands, torch's GEMM
                a = activations[0].to(backprops.dtype)
                w = (c * scale).to(backprops.dtype).view(n, *([1] * (backprops.dim() - 1)))
                rows = (backprops * w).reshape(-1, backprops.shape[-1])
                add(module.weight, rows.t().mm(a.reshape(-1, a.shape[-1])))
                if module.bias is not None:
                    add(module.bias, rows.sum(dim=0))
            elif (
                type(module) is nn.Embedding
                and module.max_norm is None
                and not module.scale_grad_by_freq
                and kernels.native_dtype(backprops.dtype)
                and backprops.is_cuda
            ):
                # every table row is the fp32 sum, over the whole batch, of the weighted backprop rows of
                # the positions that name it, written once
                total = kernels.embedding_weighted_sum(activations[0], backprops, c, module.num_embeddings, scale=scale)
                if module.padding_idx is not None:
                    total[module.padding_idx].zero_()  # autograd's embedding backward leaves that row at zero
                add(module.weight, total)
            elif type(module) is nn.Embedding and module.max_norm is None:
                ids = activations[0]
                weighted = backprops * (c * scale).to(backprops.dtype).view(n, *([1] * (backprops.dim() - 1)))
                pad = -1 if module.padding_idx is None else module.padding_idx
                add(
                    module.weight,
                    torch.ops.aten.embedding_dense_backward(
                        weighted.reshape(-1, weighted.shape[-1]),
                        ids.reshape(-1),
                        module.num_embeddings,
                        pad,
                        module.scale_grad_by_freq,
                    ),
                )
            elif (
                type(module) in (nn.Conv1d, nn.Conv2d)
                and grad_samples is None
                and not isinstance(module.padding, str)
                and module.padding_mode == "zeros"
            ):
                # the clip-weighted sum of a convolution's per-sample gradients is the ordinary
                # weight gradient for backprops weighted per sample: one weight-gradient convolution
                weighted = backprops * (c * scale).to(backprops.dtype).view(n, *([1] * (backprops.dim() - 1)))
                x = activations[0].to(backprops.dtype)
                wgrad = torch.nn.grad.conv1d_weight if type(module) is nn.Conv1d else torch.nn.grad.conv2d_weight
                if module.weight.requires_grad:
                    add(
                        module.weight,
                        wgrad(x, module.weight.shape, weighted, stride=module.stride, padding=module.padding,
                              dilation=module.dilation, groups=module.groups),
                    )
                if module.bias is not None:
                    add(module.bias, weighted.sum(dim=[0] + list(range(2, weighted.dim()))))
            else:
                if grad_samples is None:
                    grad_samples = call_sampler(self._sampler_for(module), module, activations, backprops, scale)
                for param, gs in grad_samples.items():
                    if not param.requires_grad:
                        continue
                    out = torch.empty(gs.shape[1:], device=gs.device, dtype=gs.dtype)
                    kernels.clip_accumulate([gs], c, [out], accumulate=False)
                    add(param, out)
                del grad_samples
        for param, total in sums.values():
            total = total.to(param.dtype)
            if param.grad is None:
                param.grad = total
            else:
                param.grad.add_(total)

    def log_module_gradient_sample_mode(self, module: nn.Module, *, force_functorch=False, use_ghost_clipping=True):
        """Logs, per trainable module, which of the three paths it takes (:255-290)."""
        for name, m in trainable_modules(module):
            if use_ghost_clipping and type(m) in self.NORM_SAMPLERS:
                how = "under Ghost Clipping."
            elif not force_functorch and type(m) in self.GRAD_SAMPLERS:
                how = "under Fast Gradient Clipping (hook mode)."
            else:
                how = "under Fast Gradient Clipping (functorch mode)."
            logger.info(f"Module name: {name}, module type: {type(m)}, {how}")

    @property
    def per_sample_gradient_norms(self) -> torch.Tensor:
        """Per-sample gradient norms of the last ``get_norm_sample``/``get_clipping_coef`` call."""
        if self._per_sample_gradient_norms is None:
            raise AttributeError("per_sample_gradient_norms is not set. Please call forward and backward on the model before accessing this property.")
        return self._per_sample_gradient_norms

    @per_sample_gradient_norms.setter
    def per_sample_gradient_norms(self, value):
        self._per_sample_gradient_norms = value


class GradSampleModuleFastGradientClipping(GradSampleHooksFastGradientClipping, AbstractGradSampleModule):
    """``nn.Module`` wrapper flavour of :class:`GradSampleHooksFastGradientClipping`."""

    def __init__(
        self,
        m: nn.Module,
        *,
        batch_first=True,
        loss_reduction="mean",
        strict: bool = True,
        force_functorch=False,
        max_grad_norm=1,
        use_ghost_clipping=True,
        single_backward: bool = True,
    ):
        nn.Module.__init__(self)
        GradSampleHooksFastGradientClipping.__init__(
            self,
            m,
            batch_first=batch_first,
            loss_reduction=loss_reduction,
            strict=strict,
            force_functorch=force_functorch,
            max_grad_norm=max_grad_norm,
            use_ghost_clipping=use_ghost_clipping,
            single_backward=single_backward,
        )
        self.grad_accumulation_hook = None

    def forward(self, *args, **kwargs):
        return self._module(*args, **kwargs)
