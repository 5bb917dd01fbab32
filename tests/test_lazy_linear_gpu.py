"""``GradSampleModule(..., lazy_linear_grad_sample=True)``: a Linear weight's per-sample gradient kept
as the layer's activations and backprops until somebody reads it.

What has to hold (the contracts are grad_sample/linear.py:29-51 for ``p.grad_sample`` and
optimizers/optimizer.py:432-475 for what the step makes of it): ``p.grad`` after a step equals the
materialising path's at the stated bars (fp32 1e-5, bf16 2e-2), ``p.grad_sample`` read at any
time equals the eager sampler's tensor bit for bit (the same kernel forms it), the step itself
never forms it, and a reader's in-place changes are what the step then clips and sums.
"""

import copy

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from _compare import assert_rel
from oracle import dp_oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda"
BARS = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


@pytest.fixture(scope="module")
def A():
    import opacus_amd

    return opacus_amd


class MLP(nn.Module):
    def __init__(self, d_in=96, d_h=160, d_out=10):
        super().__init__()
        self.fc1 = nn.Linear(d_in, d_h)
        self.fc2 = nn.Linear(d_h, d_out, bias=False)

    def forward(self, x):
        return self.fc2(F.gelu(self.fc1(x)))


def one_step(A, net, x, loss_of, lazy, sigma=0.0, C=0.8, opt_cls=None, seed=77, before_step=None, reduction="mean"):
    model = A.GradSampleModule(copy.deepcopy(net).to(DEV), lazy_linear_grad_sample=lazy, loss_reduction=reduction)
    g = torch.Generator(device=DEV).manual_seed(seed)
    opt = (opt_cls or A.DPOptimizer)(
        torch.optim.SGD(model.parameters(), lr=0.1), noise_multiplier=sigma, max_grad_norm=C,
        expected_batch_size=x.shape[0], generator=g, loss_reduction=reduction
    )
    opt.zero_grad()
    loss_of(model(x)).backward()
    kept = {k: p.grad_sample for k, p in model._module.named_parameters()}
    if before_step is not None:
        before_step(model)
    opt.step()
    return model, kept, {k: p.grad.clone() for k, p in model._module.named_parameters()}, g.get_offset()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("shape", [(64, 96), (24, 7, 96), (6, 3, 5, 96), (16, 32, 96)], ids=["T1", "T7", "4d", "T32"])
def test_step_from_factors_equals_the_materialising_step(A, dtype, shape):
    from opacus_amd.grad_sample.lazy import LazyLinearGradSample

    torch.manual_seed(5)
    net = MLP().to(dtype)
    x = torch.randn(*shape).to(dtype).to(DEV)
    w = torch.randn(*shape[:-1], 10).to(dtype).to(DEV)
    loss_of = lambda out: (out * w).float().flatten(1).sum(1).mean()
    _, kept_e, grads_e, _ = one_step(A, net, x, loss_of, lazy=False)
    model, kept_l, grads_l, _ = one_step(A, net, x, loss_of, lazy=True)
    for k in ("fc1.weight", "fc2.weight"):
        assert isinstance(kept_l[k], LazyLinearGradSample) and not kept_l[k].is_materialized, k  # the step never formed it
        assert kept_l[k].shape == kept_e[k].shape and kept_l[k].dtype == kept_e[k].dtype
    assert isinstance(kept_l["fc1.bias"], torch.Tensor)
    for k in grads_e:
        assert_rel(grads_l[k], grads_e[k], BARS[dtype], f"p.grad of {k}")
    # read afterwards: the eager sampler's tensor, bit for bit, and the oracle's within the bar
    for k in ("fc1.weight", "fc2.weight"):
        got = kept_l[k].materialize()
        assert torch.equal(got, kept_e[k]), k
        assert kept_l[k].is_materialized and kept_l[k].materialize() is got


def test_factors_against_the_oracle_at_sigma_zero(A):
    """Independent of the eager path: norms, clip factors and clipped mean from the CPU oracle's
    per-sample gradients of the same layer."""
    torch.manual_seed(6)
    n, T, d_in, d_out, C = 12, 9, 40, 24, 0.05
    lin = nn.Linear(d_in, d_out)
    x, w = torch.randn(n, T, d_in), torch.randn(n, T, d_out)
    model, kept, grads, _ = one_step(A, lin, x.to(DEV), lambda out: (out * w.to(DEV)).sum(), lazy=True, C=C,
                                     reduction="sum")
    gw, gb = O.linear_grad_sample(x.double(), w.double(), bias=True)
    norms = (gw.flatten(1).pow(2).sum(1) + gb.pow(2).sum(1)).sqrt()
    coef = (C / (norms + 1e-6)).clamp(max=1.0)
    assert (coef < 1).all()  # every sample clipped, so the factors matter
    assert_rel(kept["weight"].sumsq, gw.flatten(1).pow(2).sum(1), 1e-5, "squared norms from the factors")
    # a sum-reduced loss: the step leaves the clipped sum itself (optimizer.py:496-504 divides for "mean" only)
    assert_rel(grads["weight"], torch.einsum("n,nij->ij", coef, gw), 1e-5, "weight.grad")
    assert_rel(grads["bias"], torch.einsum("n,ni->i", coef, gb), 1e-5, "bias.grad")


def test_readers_get_the_tensor_and_their_changes_count(A):
    from opacus_amd import kernels
    from opacus_amd.grad_sample.lazy import LazyLinearGradSample

    torch.manual_seed(7)
    net = MLP()
    n = 32
    x = torch.randn(n, 96).to(DEV)
    y = torch.randint(0, 10, (n,)).to(DEV)
    loss_of = lambda out: F.cross_entropy(out, y)

    model = A.GradSampleModule(copy.deepcopy(net).to(DEV), lazy_linear_grad_sample=True)
    loss_of(model(x)).backward()
    gs = model._module.fc1.weight.grad_sample
    assert isinstance(gs, LazyLinearGradSample) and len(gs) == n and gs.shape == (n, 160, 96) and gs.dim() == 3
    assert gs.device.type == "cuda" and gs.dtype == torch.float32 and not gs.is_materialized  # none of that formed it
    eager = A.GradSampleModule(copy.deepcopy(net).to(DEV))
    loss_of(eager(x)).backward()
    want = eager._module.fc1.weight.grad_sample
    # a torch function, a method, an operator, an index: each sees the tensor
    assert torch.equal(torch.stack([gs, gs])[1], want)
    assert gs.is_materialized
    assert torch.equal(gs.flatten(1).norm(dim=1), want.flatten(1).norm(dim=1))
    assert torch.equal(gs * 2, want * 2) and torch.equal(gs[3], want[3]) and torch.equal(torch.cat([gs[:2], gs[2:]]), want)
    assert torch.equal(model._module.fc2.weight.grad_sample.sum(0), eager._module.fc2.weight.grad_sample.sum(0))

    # a reader that rescales the per-sample gradients in place before the step: both paths clip what it left
    def halve_odd_samples(m):
        m._module.fc1.weight.grad_sample[1::2] *= 0.5
        m._module.fc2.weight.grad_sample.mul_(3.0)

    _, _, grads_e, _ = one_step(A, net, x, loss_of, lazy=False, before_step=halve_odd_samples, C=0.3)
    _, kept, grads_l, _ = one_step(A, net, x, loss_of, lazy=True, before_step=halve_odd_samples, C=0.3)
    assert kept["fc1.weight"].is_materialized
    for k in grads_e:
        assert_rel(grads_l[k], grads_e[k], 1e-6, k)  # the same kernels on the same tensors from there on


def test_noise_stream_virtual_steps_and_per_layer_clipping(A):
    """Same generator seed: the same Philox draws land on the same elements, so the noised gradients
    differ only by the rounding of the clipped sums; a skipped (virtual) step adds into summed_grad; the
    per-layer optimizer hands each factored weight its own row of the factor table."""
    torch.manual_seed(8)
    net = MLP()
    n = 48
    x = torch.randn(n, 96).to(DEV)
    y = torch.randint(0, 10, (n,)).to(DEV)
    loss_of = lambda out: F.cross_entropy(out, y)
    _, _, ge, off_e = one_step(A, net, x, loss_of, lazy=False, sigma=1.1)
    _, kept, gl, off_l = one_step(A, net, x, loss_of, lazy=True, sigma=1.1)
    assert off_e == off_l and not kept["fc1.weight"].is_materialized
    for k in ge:
        assert (gl[k] - ge[k]).abs().max().item() <= 1e-5 * ge[k].abs().max().item(), k

    def two_microbatches(lazy):
        model = A.GradSampleModule(copy.deepcopy(net).to(DEV), lazy_linear_grad_sample=lazy)
        opt = A.DPOptimizer(torch.optim.SGD(model.parameters(), lr=0.1), noise_multiplier=0.0, max_grad_norm=0.5,
                            expected_batch_size=n)
        for i, skip in enumerate((True, False)):
            opt.zero_grad()
            F.cross_entropy(model(x[i * 24 : (i + 1) * 24]), y[i * 24 : (i + 1) * 24]).backward()
            opt.signal_skip_step(skip)
            opt.step()
        return {k: p.grad.clone() for k, p in model._module.named_parameters()}

    ve, vl = two_microbatches(False), two_microbatches(True)
    for k in ve:
        assert_rel(vl[k], ve[k], 1e-5, f"virtual steps, {k}")

    from opacus_amd.optimizers import DPPerLayerOptimizer

    kw = dict(opt_cls=DPPerLayerOptimizer, C=[0.2, 0.1, 0.3])
    _, _, pe, _ = one_step(A, net, x, loss_of, lazy=False, **kw)
    _, kept, pl, _ = one_step(A, net, x, loss_of, lazy=True, **kw)
    assert not kept["fc2.weight"].is_materialized
    for k in pe:
        assert_rel(pl[k], pe[k], 1e-5, f"per-layer clipping, {k}")

    from functools import partial

    from opacus_amd.optimizers import AdaClipDPOptimizer

    ada = partial(AdaClipDPOptimizer, target_unclipped_quantile=0.5, clipbound_learning_rate=0.2, max_clipbound=10.0,
                  min_clipbound=0.01, unclipped_num_std=1.0)
    me, _, ae, _ = one_step(A, net, x, loss_of, lazy=False, opt_cls=ada, C=0.4)
    ml, kept, al, _ = one_step(A, net, x, loss_of, lazy=True, opt_cls=ada, C=0.4)
    assert not kept["fc1.weight"].is_materialized
    for k in ae:
        assert_rel(al[k], ae[k], 1e-5, f"adaptive clipping, {k}")


def test_layers_the_option_does_not_take(A):
    """A Linear used twice in one forward pass sums its uses (grad_sample_module.py:58-59): formed at
    once. A subclass of nn.Linear, float16 and a sampler the user registered keep the eager route."""
    from opacus_amd.grad_sample.lazy import LazyLinearGradSample

    class Twice(nn.Module):
        def __init__(self):
            super().__init__()
            self.fc = nn.Linear(32, 32)
            self.head = nn.Linear(32, 4)

        def forward(self, x):
            return self.head(self.fc(torch.tanh(self.fc(x))))

    torch.manual_seed(9)
    net = Twice()
    x = torch.randn(20, 32).to(DEV)
    loss_of = lambda out: out.pow(2).sum(1).mean()
    _, ke, ge, _ = one_step(A, net, x, loss_of, lazy=False)
    _, kl, gl, _ = one_step(A, net, x, loss_of, lazy=True)
    assert isinstance(kl["fc.weight"], torch.Tensor) and isinstance(kl["head.weight"], LazyLinearGradSample)
    assert torch.equal(kl["fc.weight"], ke["fc.weight"])
    for k in ge:
        assert_rel(gl[k], ge[k], 1e-5, k)

    half = MLP().half()
    xh = torch.randn(16, 96).half().to(DEV)
    _, kh, _, _ = one_step(A, half, xh, lambda out: out.float().pow(2).sum(1).mean(), lazy=True)
    assert isinstance(kh["fc1.weight"], torch.Tensor) and kh["fc1.weight"].dtype == torch.float16


def test_full_size_headline_layer(A):
    """Linear(4096 -> 4096) at batch 128, the benchmark's layer: closed forms for an input of ones
    and backprops of 1/n (gs[n] = 1/n everywhere before clipping), and nothing of n x 64 MB formed."""
    n, d = 128, 4096
    lin = nn.Linear(d, d)
    torch.manual_seed(10)
    x = torch.randn(n, d).to(DEV)
    model = A.GradSampleModule(copy.deepcopy(lin).to(DEV), lazy_linear_grad_sample=True)
    opt = A.DPOptimizer(torch.optim.SGD(model.parameters(), lr=0.1), noise_multiplier=0.0, max_grad_norm=1.0,
                        expected_batch_size=n)
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    opt.zero_grad()
    y = torch.randn(n, d, device=DEV)
    ((model(x) - y) ** 2).sum(1).mean().backward()
    gs = model._module.weight.grad_sample
    opt.step()
    assert not gs.is_materialized
    assert torch.cuda.max_memory_allocated() - base < 2 * 1024**3  # the tensor alone would be 8.6 GB
    # against the definition on a few samples' worth of columns: b = 2 (out - y), gs[n] = b[n] a[n]^T
    with torch.no_grad():
        out = x @ lin.weight.to(DEV).t() + lin.bias.to(DEV)
        b = 2 * (out - y)
        norms = (b.double().pow(2).sum(1) * (x.double().pow(2).sum(1) + 1)).sqrt()
        coef = (1.0 / (norms + 1e-6)).clamp(max=1.0)
        want = ((coef[:, None] * b.double()).t() @ x.double()) / n
    assert_rel(model._module.weight.grad, want, 1e-5, "weight.grad at full size")
    assert_rel(gs.sumsq, b.double().pow(2).sum(1) * x.double().pow(2).sum(1), 1e-5, "closed-form squared norms")


def test_through_make_private_with_poisson_batches(A):
    """A module wrapped by the caller with the option on goes through ``PrivacyEngine.make_private``
    as any pre-wrapped module does (privacy_engine.py:171-183); Poisson batches of varying and zero
    length train, and the weights end up where the materialising run leaves them (same seeds, sigma 0)."""
    from torch.utils.data import DataLoader, TensorDataset

    def run(lazy):
        torch.manual_seed(21)
        net = MLP().to(DEV)
        wrapped = A.GradSampleModule(net, lazy_linear_grad_sample=lazy)
        ds = TensorDataset(torch.randn(40, 96), torch.randint(0, 10, (40,)))
        dl = DataLoader(ds, batch_size=4)
        engine = A.PrivacyEngine()
        model, opt, loader = engine.make_private(
            module=wrapped, optimizer=torch.optim.SGD(net.parameters(), lr=0.1), data_loader=dl, noise_multiplier=0.0,
            max_grad_norm=0.5, poisson_sampling=True,
        )
        assert model is wrapped
        torch.manual_seed(22)  # the sampler's draws
        sizes = []
        for x, y in loader:
            opt.zero_grad()
            if len(x):
                F.cross_entropy(model(x.to(DEV)), y.to(DEV)).backward()
            else:
                model(x.to(DEV)).sum().backward()
            sizes.append(len(x))
            opt.step()
        return sizes, [p.detach().clone() for p in net.parameters()]

    sizes_e, we = run(False)
    sizes_l, wl = run(True)
    assert sizes_e == sizes_l and len(set(sizes_e)) > 1
    for a, b in zip(wl, we):
        assert_rel(a, b, 1e-5, "weights after an epoch of Poisson batches")
