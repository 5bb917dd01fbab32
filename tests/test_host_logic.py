"""Host-side behaviour of the drop-in layer that needs no GPU: registry, hook bookkeeping,
guards and error paths. Arithmetic is not tested here (it has no CPU implementation: the
tests below assert that it fails loudly instead)."""

from unittest.mock import MagicMock

import math

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.utils.data import DataLoader, TensorDataset

from oracle import dp_oracle as O

import opacus_amd
from opacus_amd import (
    DPOptimizer,
    DPOptimizerFastGradientClipping,
    GradSampleHooks,
    GradSampleHooksFastGradientClipping,
    GradSampleModule,
    GradSampleModuleFastGradientClipping,
    PrivacyEngine,
    register_grad_sampler,
    register_norm_sampler,
)
from opacus_amd.grad_sample import get_gsm_class, get_hooks_class, prepare_module
from opacus_amd.optimizers import get_optimizer_class
from opacus_amd.utils.fast_gradient_clipping_utils import DPLossFastGradientClipping, DPTensorFastGradientClipping


class Scale(nn.Module):
    """A custom layer with a torch-only sampler: lets the hook machinery run on the CPU."""

    def __init__(self, d):
        super().__init__()
        self.w = nn.Parameter(torch.ones(d))

    def forward(self, x):
        return x * self.w


@register_grad_sampler(Scale)
def scale_grad_sample(layer, activations, backprops):
    prod = activations[0] * backprops
    return {layer.w: prod.reshape(prod.shape[0], -1, prod.shape[-1]).sum(1)}


@register_norm_sampler(Scale)
def scale_norm_sample(layer, activations, backprops):
    prod = activations[0] * backprops
    return {layer.w: prod.reshape(prod.shape[0], -1, prod.shape[-1]).sum(1).norm(dim=1)}


# ---- registry ---------------------------------------------------------------------------
def test_registry_writes_both_engines_and_last_wins():
    assert GradSampleHooks.GRAD_SAMPLERS[Scale] is scale_grad_sample
    assert GradSampleHooksFastGradientClipping.GRAD_SAMPLERS[Scale] is scale_grad_sample
    assert GradSampleHooksFastGradientClipping.NORM_SAMPLERS[Scale] is scale_norm_sample
    assert Scale not in getattr(GradSampleHooks, "NORM_SAMPLERS", {})

    class Tmp(nn.Module):
        pass

    @register_grad_sampler([Tmp])
    def first(layer, a, b):
        return {}

    @register_grad_sampler(Tmp)
    def second(layer, a, b):
        return {}

    assert GradSampleHooks.GRAD_SAMPLERS[Tmp] is second
    GradSampleHooks.GRAD_SAMPLERS.pop(Tmp, None)
    GradSampleHooksFastGradientClipping.GRAD_SAMPLERS.pop(Tmp, None)


def test_builtin_samplers_are_registered():
    for cls in (nn.Linear, nn.Conv1d, nn.Conv2d, nn.Embedding, nn.GroupNorm, nn.RMSNorm):
        assert cls in GradSampleHooks.GRAD_SAMPLERS
    assert set(GradSampleHooksFastGradientClipping.NORM_SAMPLERS) >= {nn.Linear, nn.Embedding}


def test_mode_tables():
    assert get_gsm_class("hooks") is GradSampleModule
    assert get_gsm_class("ghost") is GradSampleModuleFastGradientClipping
    assert get_hooks_class("hooks") is GradSampleHooks
    assert get_hooks_class("ghost") is GradSampleHooksFastGradientClipping
    with pytest.raises(NotImplementedError):
        get_gsm_class("ew")
    with pytest.raises(ValueError):
        get_gsm_class("nonsense")
    assert get_optimizer_class("flat", False, "hooks") is DPOptimizer
    assert get_optimizer_class("flat", False, "ghost") is DPOptimizerFastGradientClipping
    from opacus_amd.optimizers import AdaClipDPOptimizer, DPPerLayerOptimizer

    assert get_optimizer_class("per_layer", False, "hooks") is DPPerLayerOptimizer
    assert get_optimizer_class("adaptive", False, "hooks") is AdaClipDPOptimizer
    with pytest.raises(ValueError):
        get_optimizer_class("per_layer", False, "ghost")
    with pytest.raises(NotImplementedError):
        get_optimizer_class("flat", True, "hooks")
    with pytest.raises(ValueError):
        get_optimizer_class("weird", False, "hooks")


# ---- wrapper behaviour --------------------------------------------------------------------
def test_wrapper_surface():
    net = nn.Sequential(nn.Linear(4, 3), nn.ReLU(), nn.Linear(3, 2))
    gsm = GradSampleModule(net, autograd_weight_grads=False)
    assert all(k.startswith("_module.") for k in gsm.state_dict())
    assert gsm._module[0] is net[0]
    # per Linear: parameters off before forward, back on after it, and the capturing forward hook
    # (which hooks the output's gradient)
    assert len(net.autograd_grad_sample_hooks) == 6
    # the default keeps autograd's own weight gradients, as the reference does: one hook per layer
    with_autograd = GradSampleModule(nn.Sequential(nn.Linear(4, 3), nn.ReLU(), nn.Linear(3, 2)))
    assert with_autograd.autograd_weight_grads and len(with_autograd._module.autograd_grad_sample_hooks) == 2
    for p in net.parameters():
        assert p.grad_sample is None and p._forward_counter == 0
    with pytest.raises(ValueError, match="twice"):
        GradSampleModule(net)
    back = gsm.to_standard_module()
    assert back is net and not hasattr(net, "autograd_grad_sample_hooks")
    for p in net.parameters():
        assert not hasattr(p, "grad_sample") and not hasattr(p, "_forward_counter")
    GradSampleModule(net)  # can be wrapped again after cleanup


def test_submodule_passthrough_and_repr():
    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.fc1 = nn.Linear(2, 2)

        def forward(self, x):
            return self.fc1(x)

    gsm = GradSampleModule(Net())
    assert isinstance(gsm.fc1, nn.Linear)
    with pytest.raises(AttributeError):
        gsm.nothing_here
    assert repr(gsm).startswith("GradSampleModule(Net(")


def test_buffers_are_rejected_in_strict_mode():
    net = nn.Sequential(nn.Linear(4, 4), nn.BatchNorm1d(4))
    with pytest.raises(NotImplementedError):
        GradSampleModule(net)
    errors = GradSampleModule.validate(net, strict=False)
    assert len(errors) == 1


def test_wrap_model_false_returns_hooks_object():
    net = nn.Linear(3, 3)
    hooks = prepare_module(net, grad_sample_mode="hooks", wrap_model=False)
    assert isinstance(hooks, GradSampleHooks) and not isinstance(hooks, nn.Module)
    hooks.cleanup()
    assert not hasattr(net.weight, "grad_sample")


def test_inplace_op_on_a_hooked_output_is_fine():
    """The output-gradient hook sees the gradient with respect to the layer's own output even when
    the next op rewrites that tensor in place (a module-level full backward hook refuses this)."""

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.fc = Tmp(3, 4)

        def forward(self, x):
            return torch.relu_(self.fc(x))

    class Tmp(nn.Linear):
        pass

    seen = {}

    def sampler(layer, activations, backprops):
        seen["b"] = backprops.clone()
        return {layer.weight: torch.einsum("ni,nj->nij", backprops, activations[0]), layer.bias: backprops.clone()}

    register_grad_sampler(Tmp)(sampler)
    try:
        torch.manual_seed(0)
        net = Net()
        x = torch.randn(5, 3)
        gsm = GradSampleModule(net, loss_reduction="sum", autograd_weight_grads=True)
        out = gsm(x)
        out.sum().backward()
        want = (net.fc(x) > 0).float()  # d relu(y).sum() / dy
        assert torch.equal(seen["b"], want)
        torch.testing.assert_close(net.fc.weight.grad_sample.sum(0), net.fc.weight.grad)
        # autograd_weight_grads=False: the same per-sample gradients with the layer's parameters
        # switched off during forward, an in-place op on the re-attached output included; autograd
        # forms no weight gradient
        first = net.fc.weight.grad_sample.clone()
        gsm.remove_hooks()
        net.zero_grad()
        gsm = GradSampleModule(net, loss_reduction="sum", autograd_weight_grads=False)
        gsm(x).sum().backward()
        assert torch.equal(seen["b"], want)
        torch.testing.assert_close(net.fc.weight.grad_sample, first)
        assert net.fc.weight.grad is None and net.fc.bias.grad is None
        assert net.fc.weight.requires_grad and net.fc.bias.requires_grad
    finally:
        GradSampleHooks.GRAD_SAMPLERS.pop(Tmp, None)


def test_parameters_are_switched_back_on_whatever_happens():
    net = nn.Sequential(nn.Linear(3, 4), nn.ReLU(), nn.Linear(4, 2))
    gsm = GradSampleModule(net, autograd_weight_grads=False)
    with pytest.raises(RuntimeError):
        gsm(torch.randn(5, 7))  # wrong width: the first Linear raises inside forward
    assert all(p.requires_grad for p in net.parameters())
    assert not hasattr(net[0], "_dpk_params_off")
    # nothing is switched off without training mode, without grad mode or with hooks disabled
    gsm.eval()
    assert not gsm(torch.randn(5, 3)).requires_grad or True
    gsm.train()
    gsm.disable_hooks()
    out = gsm(torch.randn(5, 3))
    out.sum().backward()
    assert all(p.grad is not None for p in net.parameters())  # plain autograd while the hooks are off


def test_no_capture_in_eval_or_no_grad_or_disabled():
    net = Scale(3)
    gsm = GradSampleModule(net)
    x = torch.randn(2, 3)
    gsm.eval()
    gsm(x)
    assert not hasattr(net, "activations")
    gsm.train()
    with torch.no_grad():
        gsm(x)
    assert not hasattr(net, "activations")
    gsm.disable_hooks()
    gsm(x)
    assert not hasattr(net, "activations")
    gsm.enable_hooks()
    gsm(x)
    assert len(net.activations) == 1 and net.w._forward_counter == 1


# ---- hook machinery on the CPU, through a torch-only custom sampler ----------------------------
@pytest.mark.parametrize("loss_reduction", ["mean", "sum"])
@pytest.mark.parametrize("batch_first", [True, False])
def test_hook_flow_with_custom_sampler(loss_reduction, batch_first):
    torch.manual_seed(0)
    net = Scale(5)
    gsm = GradSampleModule(net, loss_reduction=loss_reduction, batch_first=batch_first)
    x = torch.randn(4, 3, 5) if batch_first else torch.randn(3, 4, 5)  # batch of 4 either way
    out = gsm(x)
    loss = out.pow(2).mean() if loss_reduction == "mean" else out.pow(2).sum()
    loss.backward()
    gs = net.w.grad_sample
    assert gs.shape == (4, 5)
    # per-sample gradients of a mean loss are those of the sum loss: they add up to n * grad
    factor = 4 if loss_reduction == "mean" else 1
    torch.testing.assert_close(gs.sum(0), net.w.grad * factor, rtol=1e-5, atol=1e-6)
    assert not hasattr(net, "max_batch_len") and net.activations == []


def test_second_backward_makes_a_list_and_zero_grad_clears():
    net = Scale(3)
    gsm = GradSampleModule(net, loss_reduction="sum")
    for _ in range(2):
        gsm(torch.randn(2, 3)).sum().backward()
    assert isinstance(net.w.grad_sample, list) and len(net.w.grad_sample) == 2
    gsm(torch.randn(2, 3)).sum().backward()
    assert len(net.w.grad_sample) == 3
    gsm.zero_grad()
    assert net.w.grad_sample is None


def test_forbid_grad_accumulation():
    net = Scale(3)
    gsm = GradSampleModule(net, loss_reduction="sum")
    gsm.forbid_grad_accumulation()
    gsm(torch.randn(2, 3)).sum().backward()
    with pytest.raises(ValueError, match="Poisson sampling is not compatible"):
        gsm(torch.randn(2, 3)).sum().backward()


def test_tied_layer_used_twice_accumulates_within_a_pass():
    net = Scale(3)

    class Twice(nn.Module):
        def __init__(self):
            super().__init__()
            self.s = net

        def forward(self, x):
            return self.s(self.s(x))

    gsm = GradSampleModule(Twice(), loss_reduction="sum")
    x = torch.randn(4, 3)
    gsm(x).sum().backward()
    gs = net.w.grad_sample
    assert isinstance(gs, torch.Tensor) and gs.shape == (4, 3)
    torch.testing.assert_close(gs.sum(0), net.w.grad)


def test_ghost_hooks_with_custom_norm_sampler_and_tying_guard():
    net = Scale(3)
    gsm = GradSampleModuleFastGradientClipping(net, loss_reduction="sum", max_grad_norm=1.0)
    x = torch.randn(4, 3)
    gsm(x).sum().backward()
    torch.testing.assert_close(net.w._norm_sample, x.norm(dim=1))
    assert net.w.grad_sample is None

    class Twice(nn.Module):
        def __init__(self):
            super().__init__()
            self.s = Scale(3)

        def forward(self, x):
            return self.s(self.s(x))

    tied = GradSampleModuleFastGradientClipping(Twice(), loss_reduction="sum")
    with pytest.raises(NotImplementedError, match="tying"):
        tied(torch.randn(2, 3))
    with pytest.raises(AttributeError):
        tied.per_sample_gradient_norms


# ---- no CPU fallback ------------------------------------------------------------------------
def test_builtin_samplers_fail_loudly_on_cpu_tensors():
    gsm = GradSampleModule(nn.Linear(4, 3), loss_reduction="sum")
    out = gsm(torch.randn(2, 4))
    with pytest.raises(RuntimeError, match="GPU only"):
        out.sum().backward()


def test_optimizer_fails_loudly_on_cpu_tensors():
    lin = nn.Linear(2, 2)
    opt = DPOptimizer(torch.optim.SGD(lin.parameters(), lr=0.1), noise_multiplier=0.0, max_grad_norm=1.0, expected_batch_size=2)
    for p in lin.parameters():
        p.grad_sample = torch.randn(2, *p.shape)
    with pytest.raises(RuntimeError, match="GPU only"):
        opt.step()


def test_missing_library_is_an_error(monkeypatch, tmp_path):
    from opacus_amd import _lib

    monkeypatch.setattr(_lib, "_LIB", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "libdpsgd_hip.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.lib()


# ---- DPOptimizer bookkeeping ------------------------------------------------------------------
def _opt(lin, **kw):
    args = dict(noise_multiplier=1.0, max_grad_norm=1.0, expected_batch_size=4)
    args.update(kw)
    return DPOptimizer(torch.optim.SGD(lin.parameters(), lr=0.1), **args)


def test_optimizer_constructor_checks_and_delegation():
    lin = nn.Linear(2, 2)
    lin.bias.requires_grad_(False)
    with pytest.raises(ValueError):
        _opt(lin, loss_reduction="max")
    with pytest.raises(ValueError):
        _opt(lin, expected_batch_size=None)
    opt = _opt(lin, expected_batch_size=None, loss_reduction="sum")
    assert opt.params == [lin.weight] and lin.weight.summed_grad is None
    assert opt.param_groups is opt.original_optimizer.param_groups
    assert opt.state is opt.original_optimizer.state and opt.defaults["lr"] == 0.1
    assert repr(opt) == repr(opt.original_optimizer)
    assert opt.state_dict() == opt.original_optimizer.state_dict()


def test_grad_sample_access_errors_and_accumulated_iterations():
    lin = nn.Linear(2, 2)
    opt = _opt(lin)
    with pytest.raises(ValueError, match="Are you using GradSampleModule"):
        opt.grad_samples
    for p in lin.parameters():
        p.grad_sample = None
    with pytest.raises(ValueError, match="not initialized"):
        opt.grad_samples
    lin.weight.grad_sample = [torch.zeros(1, 2, 2), torch.zeros(3, 2, 2)]
    lin.bias.grad_sample = torch.zeros(4, 2)
    assert opt._get_flat_grad_sample(lin.weight).shape == (4, 2, 2)
    with pytest.raises(ValueError, match="inconsistent"):
        opt.accumulated_iterations
    lin.bias.grad_sample = [torch.zeros(1, 2), torch.zeros(3, 2)]
    assert opt.accumulated_iterations == 2
    lin.bias.grad_sample = "bad"
    with pytest.raises(ValueError, match="Unexpected grad_sample type"):
        opt.grad_samples


def test_processed_flag_guard():
    from opacus_amd.optimizers.optimizer import _check_processed_flag, _mark_as_processed

    t = [torch.zeros(1), torch.zeros(1)]
    _check_processed_flag(t)
    _mark_as_processed(t)
    with pytest.raises(ValueError, match="haven't been cleared"):
        _check_processed_flag(t)
    lin = nn.Linear(2, 2)
    opt = _opt(lin)
    for p in lin.parameters():
        p.grad_sample = torch.zeros(4, *p.shape)
        _mark_as_processed(p.grad_sample)
    with pytest.raises(ValueError, match="haven't been cleared"):
        opt.clip_and_accumulate()


def test_skip_queue_and_zero_grad():
    lin = nn.Linear(2, 2)
    opt = _opt(lin)
    assert opt._check_skip_next_step() is False
    opt.signal_skip_step(True)
    opt.signal_skip_step(False)
    assert opt._check_skip_next_step(pop_next=False) is True
    assert opt._check_skip_next_step() is True and opt._check_skip_next_step() is False
    for p in lin.parameters():
        p.grad_sample = torch.zeros(4, *p.shape)
        p.summed_grad = torch.zeros_like(p)
    opt._is_last_step_skipped = True
    opt.zero_grad()
    assert lin.weight.grad_sample is None and lin.weight.summed_grad is not None
    opt._is_last_step_skipped = False
    opt.zero_grad()
    assert lin.weight.summed_grad is None


def test_batch_splitting_sampler_pieces_and_signals():
    """batch_memory_manager.py:52-69: pieces of a logical batch (numpy.array_split sizes), a skip
    signal before every piece but the last, an empty logical batch passed through with a real step."""
    import numpy as np
    from torch.utils.data import BatchSampler, DataLoader, SequentialSampler, TensorDataset

    from opacus_amd.utils.batch_memory_manager import BatchMemoryManager, BatchSplittingSampler, _split

    for total in range(1, 40):
        for m in (1, 3, 7, 16):
            want = [a.tolist() for a in np.array_split(list(range(total)), math.ceil(total / m))]
            assert _split(list(range(total)), m) == want

    class Recorder:
        def __init__(self):
            self.signals = []

        def signal_skip_step(self, do_skip=True):
            self.signals.append(do_skip)

    rec = Recorder()
    logical = [[0, 1, 2, 3, 4, 5, 6], [], [7, 8], [9, 10, 11]]
    got = list(BatchSplittingSampler(sampler=logical, max_batch_size=3, optimizer=rec))
    assert got == [[0, 1, 2], [3, 4], [5, 6], [], [7, 8], [9, 10, 11]]
    assert rec.signals == [True, True, False, False, False, False]

    ds = TensorDataset(torch.arange(20).float().unsqueeze(1))
    dl = DataLoader(ds, batch_sampler=BatchSampler(SequentialSampler(ds), batch_size=10, drop_last=False))
    rec = Recorder()
    with BatchMemoryManager(data_loader=dl, max_physical_batch_size=4, optimizer=rec) as dl2:
        assert dl2 is not dl and len(dl2.batch_sampler) == 5
        sizes = [len(b[0]) for b in dl2]
    assert sizes == [4, 3, 3, 4, 3, 3] and rec.signals == [True, True, False, True, True, False]
    with pytest.raises(ValueError):
        BatchSplittingSampler(sampler=logical, max_batch_size=0, optimizer=rec)


def test_per_layer_and_adaptive_optimizer_constructors():
    """perlayeroptimizer.py:45-47 (one bound per parameter, noise calibrated to their 2-norm) and
    adaclipoptimizer.py:71-78 (argument checks)."""
    from opacus_amd.optimizers import AdaClipDPOptimizer, DPPerLayerOptimizer

    lin = nn.Linear(3, 2)
    sgd = torch.optim.SGD(lin.parameters(), lr=0.1)
    opt = DPPerLayerOptimizer(sgd, noise_multiplier=1.0, max_grad_norm=[3.0, 4.0], expected_batch_size=4)
    assert opt.max_grad_norms == [3.0, 4.0] and opt.max_grad_norm == pytest.approx(5.0)
    with pytest.raises(ValueError):
        DPPerLayerOptimizer(sgd, noise_multiplier=1.0, max_grad_norm=[1.0], expected_batch_size=4)
    common = dict(target_unclipped_quantile=0.5, clipbound_learning_rate=0.2, max_grad_norm=1.0, expected_batch_size=4)
    with pytest.raises(ValueError, match="max_clipbound"):
        AdaClipDPOptimizer(sgd, noise_multiplier=1.0, max_clipbound=0.1, min_clipbound=0.5, unclipped_num_std=1.0, **common)
    with pytest.raises(ValueError, match="unclipped_num_std"):
        AdaClipDPOptimizer(sgd, noise_multiplier=2.0, max_clipbound=10.0, min_clipbound=0.1, unclipped_num_std=1.0, **common)
    ada = AdaClipDPOptimizer(sgd, noise_multiplier=1.0, max_clipbound=10.0, min_clipbound=0.1, unclipped_num_std=1.0, **common)
    # sigma_eff = (1 - 1/4)^(-1/2)
    assert ada._noise_std() == pytest.approx((1 - 0.25) ** -0.5)
    ada.sample_size, ada.unclipped_num = 10, 9.0  # 90 % unclipped, target 50 %: the bound shrinks
    ada.update_max_grad_norm()
    assert ada.max_grad_norm == pytest.approx(math.exp(-0.2 * 0.4))
    ada.max_grad_norm, ada.unclipped_num = 9.9, 0.0  # nothing unclipped: grows, capped at max_clipbound
    ada.update_max_grad_norm()
    assert ada.max_grad_norm == pytest.approx(10.0)


def test_no_trainable_parameters_is_a_plain_step():
    lin = nn.Linear(2, 2)
    for p in lin.parameters():
        p.requires_grad_(False)
    opt = DPOptimizer(torch.optim.SGD(lin.parameters(), lr=0.1), noise_multiplier=1.0, max_grad_norm=1.0, expected_batch_size=1)
    assert opt.pre_step() is True


def test_ghost_optimizer_is_always_one_iteration():
    lin = nn.Linear(2, 2)
    opt = DPOptimizerFastGradientClipping(
        torch.optim.SGD(lin.parameters(), lr=0.1), noise_multiplier=0.0, max_grad_norm=1.0, expected_batch_size=2
    )
    assert opt.accumulated_iterations == 1
    assert opt.clip_and_accumulate() is None and opt._get_flat_grad_sample(lin.weight) is None
    # accumulate: summed_grad shares p.grad unless a skipped step is queued
    for p in lin.parameters():
        p.grad = torch.ones_like(p)
    opt.accumulate()
    assert lin.weight.summed_grad.data_ptr() == lin.weight.grad.data_ptr()
    opt.accumulate()
    assert torch.all(lin.weight.summed_grad == 2)
    opt.zero_grad()
    opt.signal_skip_step(True)
    for p in lin.parameters():
        p.grad = torch.ones_like(p)
    assert opt.pre_step() is False and opt._is_last_step_skipped
    assert lin.weight.summed_grad.data_ptr() != lin.weight.grad.data_ptr()
    opt.zero_grad()
    assert torch.all(lin.weight.summed_grad == 1)  # survives the zero_grad of a skipped step


# ---- ghost-clipping loss wrappers ---------------------------------------------------------------
def _mock_pair(loss_reduction="mean"):
    module, optimizer = MagicMock(), MagicMock()
    module.loss_reduction = optimizer.loss_reduction = loss_reduction
    return module, optimizer


def test_dp_tensor_arithmetic_and_scalars():
    module, optimizer = _mock_pair()
    t = DPTensorFastGradientClipping(module, optimizer, torch.tensor([1.0, 2.0, 3.0]), "mean")
    assert t.item() == 2.0 and (t * 2).item() == 4.0 and (2 * t).item() == 4.0
    assert (t / 2).item() == 1.0 and (t + 1).item() == 3.0 and (1 + t).item() == 3.0
    assert (t - 1).item() == 1.0 and (5 - t).item() == 3.0 and (-t).item() == -2.0
    assert (t + t).item() == 4.0 and (t - t).item() == 0.0
    assert "DPTensorFastGradientClipping(2.0000)" == str(t) and "shape" in repr(t)
    other = DPTensorFastGradientClipping(module, optimizer, torch.tensor([1.0, 2.0, 3.0]), "sum")
    assert other.item() == 6.0
    with pytest.raises(ValueError):
        t + other


def test_dp_tensor_backward_order():
    module, optimizer = _mock_pair("sum")
    calls = []
    optimizer.zero_grad.side_effect = lambda: calls.append("zero_grad")
    module.get_clipping_coef.side_effect = lambda: (calls.append("coef"), torch.tensor([0.5, 1.0]))[1]
    module.disable_hooks.side_effect = lambda: calls.append("off")
    module.enable_hooks.side_effect = lambda: calls.append("on")
    w = torch.tensor([1.0, 1.0], requires_grad=True)
    loss = DPTensorFastGradientClipping(module, optimizer, w * torch.tensor([2.0, 3.0]), "sum")
    loss.backward()
    assert calls == ["zero_grad", "coef", "off", "on"]
    # first backward left [2, 3]; it was not zeroed by the mock; second adds coef * [2, 3]
    torch.testing.assert_close(w.grad, torch.tensor([2.0 + 1.0, 3.0 + 3.0]))


def test_adaptive_dp_tensor_updates_bound_noise_and_uses_new_bound(monkeypatch):
    """adaptive_clipping_utils.py:77-121: between the two passes the bound and the adjusted
    noise multiplier are written to module and optimizer, and the second pass is weighted with
    coefficients of the new bound."""
    from opacus_amd.utils.adaptive_clipping import DPTensorFastGradientAdaptiveClipping

    module, optimizer = _mock_pair("sum")
    module.max_grad_norm = optimizer.max_grad_norm = 1.0
    optimizer.noise_multiplier = 0.0
    norms = torch.tensor([0.5, 1.0, 2.0, 4.0] * 3)  # half unclipped at C = 1
    module.get_norm_sample.side_effect = lambda: norms
    monkeypatch.setattr(torch, "normal", lambda **kw: torch.zeros(kw["size"]))
    w = torch.ones(12, requires_grad=True)
    base = torch.arange(1.0, 13.0)
    loss = DPTensorFastGradientAdaptiveClipping(
        module, optimizer, w * base, "sum", target_unclipped_quantile=0.75, min_clipbound=0.1, max_clipbound=10.0,
        clipbound_learning_rate=0.2, initial_noise_multiplier=0.0,
    )
    assert isinstance(loss * 2, DPTensorFastGradientAdaptiveClipping) and (loss * 2).target_unclipped_quantile == 0.75
    loss.backward()
    want_bound, want_sigma, coeff = O.ghost_adaptive_update(norms, 1.0, 0.75, 0.2, 0.1, 10.0, 0.0)
    assert module.max_grad_norm == optimizer.max_grad_norm == pytest.approx(want_bound, rel=1e-12)
    assert optimizer._adjusted_noise_multiplier == want_sigma == 0.0
    torch.testing.assert_close(w.grad, base + coeff * base)  # pass 1 (not zeroed by the mock) + weighted pass 2

    # noise multiplier: the composition formula, and the batch-size guard
    module.max_grad_norm = optimizer.max_grad_norm = 1.0
    loss = DPTensorFastGradientAdaptiveClipping(module, optimizer, (w * base).detach().requires_grad_(), "sum", initial_noise_multiplier=1.0)
    loss.backward()
    assert optimizer._adjusted_noise_multiplier == pytest.approx((1.0 - (2 * 12 / 20.0) ** -2) ** -0.5, rel=1e-12)
    module.max_grad_norm = optimizer.max_grad_norm = 1.0
    with pytest.raises(AssertionError, match="Batch size is too small"):
        DPTensorFastGradientAdaptiveClipping(module, optimizer, (w * base).detach().requires_grad_(), "sum", initial_noise_multiplier=1.2).backward()
    optimizer.max_grad_norm = 2.0
    with pytest.raises(AssertionError, match="does not match"):
        DPTensorFastGradientAdaptiveClipping(module, optimizer, (w * base).detach().requires_grad_(), "sum", initial_noise_multiplier=0.0).backward()


def test_first_backward_pass_asks_for_the_entry_tensors_only():
    """The first pass of ghost clipping exists for the hooks; its weight gradients are thrown
    away. The hooks name the tensors at the start of the graph, and the pass is restricted to
    them: outputs of modules fed by tensors without grad, and leaf inputs that require grad."""
    from opacus_amd.utils.fast_gradient_clipping_utils import first_pass_backward

    def forget_forward(module):  # what the backward hooks would have done, without kernels
        for m in module.modules():
            m.__dict__.pop("activations", None)
        for p in module.parameters():
            p._forward_counter = 0

    net = nn.Sequential(nn.Linear(4, 5), nn.Tanh(), nn.Linear(5, 3), nn.Tanh(), nn.Linear(3, 2))
    ghost = GradSampleModuleFastGradientClipping(net)
    ghost.disable_hooks()
    ghost(torch.randn(2, 4))
    assert ghost.first_backward_inputs() == []
    ghost.enable_hooks()
    fired = []
    ghost.capture_backprops_hook = lambda module, *a, **k: fired.append(module)
    out = ghost(torch.randn(2, 4))
    leaves = ghost.first_backward_inputs()
    assert len(leaves) == 1 and leaves[0].shape == (2, 5) and not leaves[0].is_leaf  # the first Linear's output
    assert ghost.first_backward_inputs() == []  # consumed
    # the restricted pass reaches every hooked layer's output, forms no weight gradient and
    # leaves no gradient behind on the activation it was asked for
    ghost.first_backward_inputs = lambda: leaves
    first_pass_backward(ghost, out.sum())
    assert fired == [net[4], net[2], net[0]]
    assert all(p.grad is None for p in net.parameters()) and leaves[0].grad is None
    del ghost.first_backward_inputs
    # an in-place op on the entry layer's output: its parameters are asked for instead
    forget_forward(net)
    ghost.remove_hooks()
    inplace = nn.Sequential(net[0], nn.ReLU(inplace=True), net[2])
    ghost1 = GradSampleModuleFastGradientClipping(inplace)
    ghost1.capture_backprops_hook = lambda *a, **k: None
    ghost1(torch.randn(2, 4))
    assert {id(t) for t in ghost1.first_backward_inputs()} == {id(net[0].weight), id(net[0].bias)}
    # a frozen entry layer moves the entry to the next trainable module; a leaf input that
    # requires grad is a tensor to reach as well
    net[0].weight.requires_grad_(False)
    net[0].bias.requires_grad_(False)
    forget_forward(net)
    ghost1.remove_hooks()
    ghost2 = GradSampleModuleFastGradientClipping(nn.Sequential(net[0], net[1], net[2]))
    ghost2.capture_backprops_hook = lambda *a, **k: None
    x = torch.randn(2, 4)
    ghost2(x)
    (leaf,) = ghost2.first_backward_inputs()
    assert leaf.shape == (2, 3)  # the second Linear's output
    forget_forward(net)
    x.requires_grad_(True)
    ghost2(x)
    assert {id(t) for t in ghost2.first_backward_inputs()} == {id(x)}  # seen at the model's entrance
    forget_forward(net)
    ghost2(x * 2.0)  # a computed input has leaves of its own: no restriction
    assert ghost2.first_backward_inputs() == []
    # a module object without the method (or a mock) falls back to the plain pass
    w = torch.ones(3, requires_grad=True)
    first_pass_backward(object(), (w * 2).sum())
    torch.testing.assert_close(w.grad, torch.full((3,), 2.0))


def test_single_pass_guard_sees_uses_of_parameters_outside_the_hooked_layers():
    """The single backward pass rebuilds the clipped sum from the hooked layers alone; the
    reference's second pass differentiates the whole graph (fast_gradient_clipping_utils.py:193-201).
    ``single_pass_is_exact`` compares the uses of every trainable parameter that autograd recorded
    with the layer calls that the forward hooks counted, and ``backward()`` takes two passes when
    they differ."""
    torch.manual_seed(0)

    def forget_forward(module):
        for m in module.modules():
            m.__dict__.pop("activations", None)
        for p in module.parameters():
            p._forward_counter = 0

    class TwoUses(nn.Module):
        def __init__(self):
            super().__init__()
            self.fc1, self.ln, self.fc2 = nn.Linear(4, 6), nn.LayerNorm(6), nn.Linear(6, 3)

        def forward(self, x):
            return self.fc2(self.ln(torch.tanh(self.ln(self.fc1(x)))))  # one layer applied twice

    net = TwoUses()
    ghost = GradSampleModuleFastGradientClipping(net)
    x = torch.randn(5, 4)
    loss = ghost(x).pow(2).sum(1)
    assert ghost.single_pass_is_exact(loss.mean())
    # a regulariser on the weights is a use that no hook has seen
    assert not ghost.single_pass_is_exact((loss + 0.1 * net.fc1.weight.pow(2).sum()).mean())
    assert not ghost.single_pass_is_exact((loss + 1e-3 * sum(p.pow(2).sum() for p in net.parameters())).mean())
    # so is a functional use of a hooked layer's weight beside the layer's own call
    assert not ghost.single_pass_is_exact((loss + F.linear(x, net.fc1.weight).sum(1)).mean())
    # and a trainable parameter that belongs to no layer of the wrapped module
    outside = nn.Parameter(torch.ones(()))
    assert not ghost.single_pass_is_exact((loss * outside).mean())
    # tensors that are not parameters (an input that requires grad) do not count
    xg = torch.randn(5, 4, requires_grad=True)
    forget_forward(net)
    assert ghost.single_pass_is_exact(ghost(xg).pow(2).sum(1).mean())
    # a frozen parameter may be used anywhere
    forget_forward(net)
    net.fc2.bias.requires_grad_(False)
    ghost.remove_hooks()
    ghost = GradSampleModuleFastGradientClipping(net)
    loss = ghost(x).pow(2).sum(1)
    assert ghost.single_pass_is_exact((loss + net.fc2.bias.sum()).mean())
    assert ghost.single_pass_is_exact(torch.zeros(()))  # no graph at all

    # backward(): an inexact step is run with two passes (single_backward is off while its hooks fire)
    module, optimizer = _mock_pair("sum")
    module.single_backward = True
    module.single_pass_is_exact.side_effect = lambda reduced: False
    seen = []
    module.get_clipping_coef.side_effect = lambda: (seen.append(module.single_backward), torch.tensor([0.5, 1.0]))[1]
    w = torch.tensor([1.0, 1.0], requires_grad=True)
    with pytest.warns(UserWarning, match="two backward passes"):
        DPTensorFastGradientClipping(module, optimizer, w * torch.tensor([2.0, 3.0]), "sum").backward()
    assert seen == [False] and module.single_backward is True
    module.accumulate_clipped_gradients.assert_not_called()
    torch.testing.assert_close(w.grad, torch.tensor([2.0 + 1.0, 3.0 + 3.0]))  # both passes ran (the mock zeroes nothing)
    # an exact step takes the single pass
    module.single_pass_is_exact.side_effect = lambda reduced: True
    DPTensorFastGradientClipping(module, optimizer, w * torch.tensor([2.0, 3.0]), "sum").backward()
    module.accumulate_clipped_gradients.assert_called_once()


def test_dp_loss_requires_consistent_reductions_and_restores_reduction():
    module, optimizer = _mock_pair("mean")
    crit = nn.CrossEntropyLoss(reduction="mean")
    with pytest.raises(AssertionError):
        DPLossFastGradientClipping(module, optimizer, nn.CrossEntropyLoss(reduction="sum"), "mean")
    with pytest.raises(AssertionError):
        DPLossFastGradientClipping(module, optimizer, crit, "max")
    dpl = DPLossFastGradientClipping(module, optimizer, crit, "mean")
    logits, y = torch.randn(6, 5), torch.randint(0, 5, (6,))
    out = dpl(logits, y)
    assert crit.reduction == "mean" and out.loss_per_sample.shape == (6,)
    torch.testing.assert_close(out.detach(), F.cross_entropy(logits, y))


@pytest.mark.parametrize("loss_reduction", ["mean", "sum"])
def test_dp_loss_sequence_shape_and_ignore_index(loss_reduction):
    module, optimizer = _mock_pair(loss_reduction)
    crit = nn.CrossEntropyLoss(reduction=loss_reduction, ignore_index=-100)
    dpl = DPLossFastGradientClipping(module, optimizer, crit, loss_reduction)
    B, T, V = 3, 4, 7
    logits = torch.randn(B * T, V)
    y = torch.randint(0, V, (B * T,))
    y[1] = y[5] = y[6] = -100
    out = dpl(logits, y, shape=(B, T, V))
    assert out.loss_per_sample.shape == (B,)
    tok = F.cross_entropy(logits, y, reduction="none", ignore_index=-100).view(B, T)
    if loss_reduction == "sum":
        want = tok.sum(1)
    else:
        want = tok.sum(1) / (y.view(B, T) != -100).sum(1).clamp(min=1)
    torch.testing.assert_close(out.loss_per_sample, want)


# ---- PrivacyEngine wiring -----------------------------------------------------------------------
def _loader(n=8, bs=4):
    return DataLoader(TensorDataset(torch.randn(n, 4), torch.randint(0, 2, (n,))), batch_size=bs)


def test_make_private_arity_and_wiring():
    with pytest.warns(UserWarning, match="Secure RNG turned off"):
        engine = PrivacyEngine()
    net = nn.Linear(4, 2)
    sgd = torch.optim.SGD(net.parameters(), lr=0.1)
    model, opt, dl = engine.make_private(
        module=net, optimizer=sgd, data_loader=_loader(), noise_multiplier=1.1, max_grad_norm=1.0, poisson_sampling=False
    )
    assert isinstance(model, GradSampleModule) and type(opt) is DPOptimizer
    assert opt.expected_batch_size == 4 and opt.noise_multiplier == 1.1 and opt.step_hook is not None
    opt.step_hook(MagicMock(noise_multiplier=1.1, accumulated_iterations=1))
    opt.step_hook(MagicMock(noise_multiplier=1.1, accumulated_iterations=1))
    assert engine.accountant.history == [(1.1, 0.5, 2)] and len(engine.accountant) == 2

    net2 = nn.Linear(4, 2)
    out = PrivacyEngine().make_private(
        module=net2,
        optimizer=torch.optim.SGD(net2.parameters(), lr=0.1),
        data_loader=_loader(),
        noise_multiplier=1.0,
        max_grad_norm=2.0,
        poisson_sampling=False,
        grad_sample_mode="ghost",
    )
    assert len(out) == 4
    model, opt, crit, dl = out
    assert isinstance(model, GradSampleModuleFastGradientClipping) and model.max_grad_norm == 2.0
    assert type(opt) is DPOptimizerFastGradientClipping and isinstance(crit, DPLossFastGradientClipping)


def test_make_private_errors():
    net, other = nn.Linear(4, 2), nn.Linear(4, 2)
    engine = PrivacyEngine()
    common = dict(data_loader=_loader(), noise_multiplier=1.0, max_grad_norm=1.0)
    with pytest.raises(ValueError, match="Module parameters are different"):
        engine.make_private(module=net, optimizer=torch.optim.SGD(other.parameters(), lr=0.1), poisson_sampling=False, **common)
    wrapped = GradSampleModule(net, loss_reduction="sum")
    with pytest.raises(ValueError, match="Pre-existing GradSampleModule"):
        engine.make_private(module=wrapped, optimizer=torch.optim.SGD(net.parameters(), lr=0.1), poisson_sampling=False, **common)
    wrapped.to_standard_module()
    hooks_obj, opt, _ = engine.make_private(
        module=net, optimizer=torch.optim.SGD(net.parameters(), lr=0.1), poisson_sampling=False, wrap_model=False, **common
    )
    assert isinstance(hooks_obj, GradSampleHooks) and not isinstance(hooks_obj, nn.Module)


def test_secure_mode_is_not_reproducible_from_any_seed():
    """privacy_engine.py:86-96 builds a generator over /dev/urandom and refuses seeds. Here: noise keys
    come from os.urandom per launch, the sampling generator is seeded from os.urandom, a seed or a noise
    generator is refused, and the construction says that the generators are not cryptographic."""
    from opacus_amd.optimizers.optimizer import _NOISE_KEY_DOMAIN, philox_stream

    dev = torch.device("cuda", 0)
    torch.manual_seed(5)
    a = philox_stream(None, dev, secure=True)
    torch.manual_seed(5)
    b = philox_stream(None, dev, secure=True)
    assert a != b and all(0 <= v < 2**64 for v in a + b)
    g = torch.Generator().manual_seed(3)
    c = philox_stream(g, dev, secure=True)
    assert g.initial_seed() == 3 and c != a  # the caller's generator is not consulted
    assert torch.equal(torch.Generator().manual_seed(3).get_state(), g.get_state())
    # non-secure: a CPU generator gives repeatable keys
    k1 = philox_stream(torch.Generator().manual_seed(3), dev)
    k2 = philox_stream(torch.Generator().manual_seed(3), dev)
    assert k1 == k2 and _NOISE_KEY_DOMAIN != 0

    # the reference's flag asks for a CSPRNG, which is not there: refused as the reference refuses
    # without torchcsprng (privacy_engine.py:86-96); the weaker mode has to be named
    with pytest.raises(ImportError, match="urandom-philox"):
        PrivacyEngine(secure_mode=True)
    with pytest.raises(ValueError):
        PrivacyEngine(secure_mode="yes")
    with pytest.warns(UserWarning, match="not cryptographically secure"):
        e1 = PrivacyEngine(secure_mode="urandom-philox")
    with pytest.warns(UserWarning, match="os.urandom"):
        e2 = PrivacyEngine(secure_mode=PrivacyEngine.SECURE_MODE_URANDOM_PHILOX)
    assert e1.secure_rng is not None and e1.secure_rng.initial_seed() != e2.secure_rng.initial_seed()
    net = nn.Linear(4, 2)
    sgd = torch.optim.SGD(net.parameters(), lr=0.1)
    with pytest.raises(ValueError, match="prohibited in secure mode"):
        e1.make_private(
            module=net, optimizer=sgd, data_loader=_loader(), noise_multiplier=1.0, max_grad_norm=1.0,
            noise_generator=torch.Generator(), poisson_sampling=False,
        )
    _, opt, dl = e1.make_private(
        module=net, optimizer=sgd, data_loader=_loader(), noise_multiplier=1.0, max_grad_norm=1.0, poisson_sampling=True
    )
    assert opt.secure_mode and opt.generator is e1.secure_rng
    assert dl.batch_sampler.generator is e1.secure_rng


def test_poisson_sampler_and_empty_batches():
    """uniform_sampler.py:22-70 and data_loader.py:30-147: independent inclusion with probability
    ``sample_rate``, ``int(1 / sample_rate)`` batches per epoch, reproducible from the generator; an
    empty draw is collated into tensors with a batch dimension of zero."""
    from opacus_amd.data_loader import DPDataLoader, wrap_collate_with_empty
    from opacus_amd.utils.uniform_sampler import UniformWithReplacementSampler

    g = torch.Generator().manual_seed(0)
    sampler = UniformWithReplacementSampler(num_samples=1000, sample_rate=0.1, generator=g)
    batches = list(sampler)
    assert len(batches) == len(sampler) == 10
    sizes = torch.tensor([len(b) for b in batches], dtype=torch.float64)
    assert abs(sizes.mean().item() - 100) < 4 * (90 / 10) ** 0.5  # Binomial(1000, 0.1), ten draws
    assert all(b == sorted(set(b)) and 0 <= b[0] and b[-1] < 1000 for b in batches)
    again = list(UniformWithReplacementSampler(num_samples=1000, sample_rate=0.1, generator=torch.Generator().manual_seed(0)))
    assert again == batches
    with pytest.raises(ValueError):
        UniformWithReplacementSampler(num_samples=0, sample_rate=0.5)

    from torch.utils.data._utils.collate import default_collate

    collate = wrap_collate_with_empty(
        collate_fn=default_collate, sample_empty_shapes=[(0, 4), (0,)], dtypes=[torch.float32, torch.int64]
    )
    first_empty = collate([])
    assert [tuple(t.shape) for t in first_empty] == [(0, 4), (0,)] and first_empty[1].dtype == torch.int64
    full = collate([(torch.ones(4), torch.tensor(1)), (torch.zeros(4), torch.tensor(0))])
    assert full[0].shape == (2, 4)
    empty = collate([])
    assert type(empty) is type(full) and empty[0].shape == (0, 4) and empty[1].shape == (0,) and empty[1].dtype == torch.int64
    rnd = wrap_collate_with_empty(collate_fn=default_collate, rand_on_empty=True)
    rnd([(torch.ones(4), torch.tensor(1))])
    assert rnd([])[0].shape == (1, 4)
    nested = wrap_collate_with_empty(collate_fn=None)
    nested({"x": torch.ones(3, 2), "y": [torch.ones(3)]})
    e = nested([])
    assert e["x"].shape == (0, 2) and e["y"][0].shape == (0,)
    bad = wrap_collate_with_empty(collate_fn=None)
    bad(["text"])
    with pytest.raises(TypeError):
        bad([])

    base = _loader(n=64, bs=8)
    dp = DPDataLoader.from_data_loader(base, generator=torch.Generator().manual_seed(1))
    assert dp.sample_rate == 1 / 8 and len(dp) == 8
    seen = [len(y) for _, y in dp]
    assert len(seen) == 8 and len(set(seen)) > 1  # sizes vary


def test_make_private_with_poisson_sampling_is_the_default():
    net = nn.Linear(4, 2)
    model, opt, dl = PrivacyEngine().make_private(
        module=net, optimizer=torch.optim.SGD(net.parameters(), lr=0.1), data_loader=_loader(n=32, bs=4),
        noise_multiplier=1.0, max_grad_norm=1.0,
    )
    from opacus_amd.data_loader import DPDataLoader

    assert isinstance(dl, DPDataLoader) and dl.sample_rate == 1 / 8 and opt.expected_batch_size == 4
    assert model.grad_accumulation_allowed is False  # privacy_engine.py:429-430


@pytest.mark.parametrize("kind", ["lstm", "gru", "rnn_tanh", "rnn_relu"])
def test_recurrent_layers_equal_torch_modules_and_share_their_state_dict(kind):
    """opacus/tests/dp_layers/dp_rnn_test.py: same parameter names, state dict loadable both ways,
    same outputs and final states as torch.nn for tensors and packed sequences (unsorted lengths,
    initial states), over layers x directions x batch_first x bias. Forward only: no kernel runs."""
    from torch.nn.utils.rnn import pack_padded_sequence

    from opacus_amd.layers import DPGRU, DPLSTM, DPRNN

    DP, NN, kw = {
        "lstm": (DPLSTM, nn.LSTM, {}),
        "gru": (DPGRU, nn.GRU, {}),
        "rnn_tanh": (DPRNN, nn.RNN, {"nonlinearity": "tanh"}),
        "rnn_relu": (DPRNN, nn.RNN, {"nonlinearity": "relu"}),
    }[kind]
    torch.manual_seed(5)
    for layers, bi, bf, bias in [(1, False, False, True), (2, True, True, True), (2, True, False, False), (1, True, True, False)]:
        ref = NN(5, 7, num_layers=layers, bidirectional=bi, batch_first=bf, bias=bias, **kw).double()
        dp = DP(5, 7, num_layers=layers, bidirectional=bi, batch_first=bf, bias=bias, **kw).double()
        assert [k for k, _ in dp.named_parameters()] == [k for k, _ in ref.named_parameters()]
        assert list(dp.state_dict()) == list(ref.state_dict())
        dp.load_state_dict(ref.state_dict())
        ref.load_state_dict(dp.state_dict())
        B, T = 4, 6
        x = torch.randn(B, T, 5).double() if bf else torch.randn(T, B, 5).double()
        h0 = torch.randn(layers * (2 if bi else 1), B, 7).double()
        state = (h0, torch.randn_like(h0)) if kind == "lstm" else h0
        for inp in (x, pack_padded_sequence(x, torch.tensor([3, 6, 1, 4]), batch_first=bf, enforce_sorted=False)):
            for st in (None, state):
                o1, s1 = ref(inp, st)
                o2, s2 = dp(inp, st)
                if isinstance(o1, torch.nn.utils.rnn.PackedSequence):
                    assert torch.equal(o1.batch_sizes, o2.batch_sizes) and torch.equal(o1.sorted_indices, o2.sorted_indices)
                    o1, o2 = o1.data, o2.data
                torch.testing.assert_close(o2, o1, rtol=1e-10, atol=1e-12)
                for a, b in zip(s1 if isinstance(s1, tuple) else (s1,), s2 if isinstance(s2, tuple) else (s2,)):
                    torch.testing.assert_close(b, a, rtol=1e-10, atol=1e-12)
    with pytest.raises(NotImplementedError):
        DP(5, 7, proj_size=2, **kw)
    with pytest.raises(ValueError):
        DP(5, 7, dropout=1.5, **kw)


def test_recurrent_layers_get_hooks_on_their_linear_maps_only():
    from opacus_amd.layers import DPLSTM, RNNLinear

    gsm = GradSampleModule(nn.Sequential(DPLSTM(4, 3, num_layers=2, bidirectional=True)))
    hooked = list(gsm.iterate_submodules(gsm._module))
    assert len(hooked) == 8 and all(type(m) is RNNLinear for m in hooked)
    assert len(list(gsm.parameters())) == 16  # four cells x (ih, hh) x (weight, bias), each listed once


@pytest.mark.parametrize("batch_first", [False, True])
def test_multihead_attention_equals_torch_module_and_shares_its_state_dict(batch_first):
    """opacus/tests/dp_layers/dp_multihead_attention_test.py: outputs and averaged weights of
    torch.nn.MultiheadAttention from its own state dict (and back, same keys in the same order),
    over bias / add_bias_kv / add_zero_attn / kdim, vdim / masks, with and without the weights."""
    from opacus_amd.layers import DPMultiheadAttention

    torch.manual_seed(8)
    N, L, S = 3, 5, 7
    for bias, kv, zero, kdim, vdim in [(True, False, False, None, None), (False, True, True, None, None), (True, True, False, 6, 10)]:
        ref = nn.MultiheadAttention(8, 2, bias=bias, add_bias_kv=kv, add_zero_attn=zero, kdim=kdim, vdim=vdim, batch_first=batch_first).double()
        dp = DPMultiheadAttention(8, 2, bias=bias, add_bias_kv=kv, add_zero_attn=zero, kdim=kdim, vdim=vdim, batch_first=batch_first).double()
        dp.load_state_dict(ref.state_dict())
        assert list(dp.state_dict()) == list(ref.state_dict())
        ref.load_state_dict(dp.state_dict())
        shape = (lambda T, E: (N, T, E)) if batch_first else (lambda T, E: (T, N, E))
        q, k, v = (torch.randn(*shape(T, E)).double() for T, E in ((L, 8), (S, kdim or 8), (S, vdim or 8)))
        kpm = torch.zeros(N, S, dtype=torch.bool)
        kpm[1, -2:] = True
        am = torch.rand(L, S) > 0.8
        am[:, 0] = False
        for kwargs in ({}, {"key_padding_mask": kpm}, {"attn_mask": am}, {"attn_mask": torch.randn(L, S).double()}):
            o1, w1 = ref(q, k, v, **kwargs)
            o2, w2 = dp(q, k, v, **kwargs)
            torch.testing.assert_close(o2, o1, rtol=1e-9, atol=1e-11)
            torch.testing.assert_close(w2, w1, rtol=1e-9, atol=1e-11)
            o3, w3 = dp(q, k, v, need_weights=False, **kwargs)
            assert w3 is None
            torch.testing.assert_close(o3, o1, rtol=1e-7, atol=1e-9)
    with pytest.raises(AssertionError):
        dp(q, k, v, is_causal=True)


def test_package_surface():
    for name in opacus_amd.__all__:
        assert hasattr(opacus_amd, name)


# ---- bench.py command line ------------------------------------------------------------------------
def test_bench_refuses_more_than_one_gpu():
    """One GPU is all this build measures: a larger --gpus must end at once with a message
    that says so, before anything touches a device."""
    import subprocess
    import sys
    from pathlib import Path

    bench = Path(__file__).resolve().parents[1] / "bench.py"
    done = subprocess.run([sys.executable, str(bench), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert done.returncode != 0
    assert "one GPU" in (done.stdout + done.stderr)


def test_lazy_linear_grad_sample_answers_what_it_can_without_the_tensor(monkeypatch):
    """The stand-in for a Linear weight's per-sample gradient (grad_sample/linear.py:41-48 kept as its
    two factors): shape questions, the optimizer's processed flag and the hooks' filing must not
    form the [n, out, in] tensor; a second result for the same parameter in one pass must."""
    from opacus_amd.grad_sample import grad_sample_module as gsm
    from opacus_amd.grad_sample.lazy import LazyLinearGradSample
    from opacus_amd.optimizers import optimizer as optmod

    formed = []

    def fake_materialize(self):
        formed.append(self)
        if self._gs is None:
            self._gs = self._scale * torch.einsum("n...i,n...j->nij", self._b, self._a)
        return self._gs

    monkeypatch.setattr(LazyLinearGradSample, "materialize", fake_materialize)
    b, a = torch.randn(5, 3, 4), torch.randn(5, 3, 6)
    lz = LazyLinearGradSample(b, a, scale=2.0)
    assert lz.shape == (5, 4, 6) and len(lz) == 5 and lz.dim() == 3 and lz.numel() == 120 and lz.size(1) == 4
    assert lz.dtype == torch.float32 and lz.device.type == "cpu" and "factors only" in repr(lz)
    optmod._check_processed_flag(lz)
    optmod._mark_as_processed(lz)
    with pytest.raises(ValueError, match="haven't been cleared"):
        optmod._check_processed_flag(lz)
    p = nn.Parameter(torch.zeros(4, 6))
    gsm.create_or_accumulate_grad_sample(param=p, grad_sample=lz, max_batch_len=5)
    assert p._current_grad_sample is lz and not formed
    # everything else is the tensor's business
    want = 2.0 * torch.einsum("nti,ntj->nij", b, a)
    torch.testing.assert_close(torch.stack([lz])[0], want)
    assert formed
    torch.testing.assert_close(lz.flatten(1).sum(1), want.flatten(1).sum(1))
    torch.testing.assert_close((lz * 2)[1], 2 * want[1])
    # a second use of the layer in the same pass adds into the first: both formed
    other = LazyLinearGradSample(torch.randn(5, 3, 4), torch.randn(5, 3, 6))
    first = LazyLinearGradSample(b, a, scale=2.0)
    q = nn.Parameter(torch.zeros(4, 6))
    gsm.create_or_accumulate_grad_sample(param=q, grad_sample=first, max_batch_len=5)
    gsm.create_or_accumulate_grad_sample(param=q, grad_sample=other, max_batch_len=5)
    assert isinstance(q._current_grad_sample, torch.Tensor)
    torch.testing.assert_close(q._current_grad_sample, want + torch.einsum("nti,ntj->nij", other._b, other._a))
    # a batch shorter than the longest of the pass goes into the zero-filled buffer as before
    r = nn.Parameter(torch.zeros(4, 6))
    gsm.create_or_accumulate_grad_sample(param=r, grad_sample=LazyLinearGradSample(b[:3], a[:3]), max_batch_len=5)
    assert r._current_grad_sample.shape == (5, 4, 6) and not r._current_grad_sample[3:].any()
