"""Pins the CPU oracle before anything is compared against it.

Every oracle function is checked against something it does not share code with: the
reference's golden vectors, batch-of-one autograd (the reference's own microbatch
method), library routines (F.unfold, F.conv2d's autograd), closed forms, or known-answer
vectors. A dropped term, a swapped operand or a wrong index fails at least one of these.
"""

import math

import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import dp_oracle as O


def _per_sample_autograd(module, x, loss_fn):
    """grad of loss_fn(module(x[i:i+1])) for each i, stacked: brute force."""
    out = {k: [] for k, _ in module.named_parameters()}
    for i in range(x.shape[0]):
        module.zero_grad()
        loss_fn(module(x[i : i + 1])).backward()
        for k, p in module.named_parameters():
            out[k].append(p.grad.clone())
    module.zero_grad()
    return {k: torch.stack(v) for k, v in out.items()}


def _backprops(module, x, loss_fn):
    """(activation, d loss / d output) of a single-layer module for a sum loss."""
    y = module(x)
    y.retain_grad()
    loss_fn(y).backward()
    return y.grad.detach()


# ---- Linear ---------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(5, 7), (4, 3, 7), (3, 2, 5, 7)])
def test_linear_grad_sample_vs_microbatch(shape):
    torch.manual_seed(0)
    lin = nn.Linear(7, 6).double()
    x = torch.randn(*shape, dtype=torch.float64)
    w = torch.randn(6, dtype=torch.float64)
    loss = lambda y: (y * w).pow(2).sum()  # noqa: E731
    b = _backprops(lin, x, loss)
    gs_w, gs_b = O.linear_grad_sample(x, b)
    want = _per_sample_autograd(lin, x, loss)
    torch.testing.assert_close(gs_w, want["weight"], rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(gs_b, want["bias"], rtol=1e-12, atol=1e-12)
    # weight gradient is [out, in], not its transpose
    assert gs_w.shape == (shape[0], 6, 7)


def test_linear_grad_sample_microbatch_helper_agrees():
    torch.manual_seed(1)
    lin = nn.Linear(5, 3).double()
    x = torch.randn(6, 4, 5, dtype=torch.float64)
    mb = O.microbatch_grad_sample(lin, x, loss_reduction="sum")
    y = lin(x)
    y.retain_grad()
    nn.L1Loss(reduction="sum")(y, torch.zeros_like(y)).backward()
    gs_w, gs_b = O.linear_grad_sample(x, y.grad)
    torch.testing.assert_close(gs_w, mb["weight"])
    torch.testing.assert_close(gs_b, mb["bias"])


@pytest.mark.parametrize("T", [1, 2, 9])
def test_linear_norm_sample_equals_norm_of_grad_sample(T):
    torch.manual_seed(2)
    a = torch.randn(5, T, 11, dtype=torch.float64)
    b = torch.randn(5, T, 7, dtype=torch.float64)
    gs_w, gs_b = O.linear_grad_sample(a, b)
    nw, nb = O.linear_norm_sample(a, b)
    torch.testing.assert_close(nw, gs_w.flatten(1).norm(dim=1), rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(nb, gs_b.norm(dim=1), rtol=1e-10, atol=1e-12)


def test_linear_norm_sample_2d_closed_form_and_rank_gap():
    torch.manual_seed(3)
    a = torch.randn(4, 6, dtype=torch.float64)
    b = torch.randn(4, 3, dtype=torch.float64)
    nw, nb = O.linear_norm_sample(a, b)
    torch.testing.assert_close(nw, a.norm(dim=1) * b.norm(dim=1))
    torch.testing.assert_close(nb, b.norm(dim=1))
    # 4-d backprops: the reference returns nothing
    assert O.linear_norm_sample(torch.randn(2, 2, 2, 6), torch.randn(2, 2, 2, 3)) == (None, None)


# ---- Conv2d ---------------------------------------------------------------------------
CONV_CASES = [
    dict(C=3, O=4, k=(3, 3), stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=1, H=6, W=7),
    dict(C=4, O=6, k=(3, 2), stride=(2, 1), padding=(0, 2), dilation=(1, 2), groups=2, H=9, W=8),
    dict(C=2, O=2, k=(2, 3), stride=(1, 2), padding="same", dilation=(2, 1), groups=1, H=7, W=9),
    dict(C=6, O=3, k=(1, 1), stride=(1, 1), padding="valid", dilation=(1, 1), groups=3, H=4, W=4),
    dict(C=1, O=16, k=(8, 8), stride=(2, 2), padding=(3, 3), dilation=(1, 1), groups=1, H=28, W=28),
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_unfold2d_equals_F_unfold_exactly(case):
    torch.manual_seed(4)
    x = torch.randn(3, case["C"], case["H"], case["W"])
    # F.unfold has no "same": the input is padded by hand with the amounts unfold2d must use
    pt, pb, pl, pr = O.conv2d_padding(case["padding"], case["k"], case["dilation"])
    want = F.unfold(F.pad(x, (pl, pr, pt, pb)), kernel_size=case["k"], stride=case["stride"], dilation=case["dilation"])
    got = O.unfold2d(x, kernel_size=case["k"], padding=case["padding"], stride=case["stride"], dilation=case["dilation"])
    torch.testing.assert_close(got, want, rtol=0, atol=0)


def test_same_padding_puts_smaller_half_first():
    assert O.conv2d_padding("same", (2, 4), (1, 1)) == (0, 1, 1, 2)
    assert O.conv2d_padding("same", (3, 3), (2, 1)) == (2, 2, 1, 1)
    assert O.conv2d_padding((1, 2), (3, 3), (1, 1)) == (1, 1, 2, 2)


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d_grad_sample_vs_microbatch(case):
    torch.manual_seed(5)
    stride = case["stride"]
    if case["padding"] == "same" and stride != (1, 1):
        # nn.Conv2d refuses padding="same" with a stride; check the oracle through explicit padding
        pt, pb, pl, pr = O.conv2d_padding("same", case["k"], case["dilation"])
        conv = nn.Conv2d(case["C"], case["O"], case["k"], stride, 0, case["dilation"], case["groups"]).double()
        pad = lambda t: F.pad(t, (pl, pr, pt, pb))  # noqa: E731
        mod = lambda t: conv(pad(t))  # noqa: E731
    else:
        conv = nn.Conv2d(case["C"], case["O"], case["k"], stride, case["padding"], case["dilation"], case["groups"]).double()
        mod = conv
    x = torch.randn(3, case["C"], case["H"], case["W"], dtype=torch.float64)
    loss = lambda y: y.pow(3).sum()  # noqa: E731

    y = mod(x)
    y.retain_grad()
    loss(y).backward()
    b = y.grad.detach()
    conv.zero_grad()
    gs_w, gs_b = O.conv2d_grad_sample(
        x, b, kernel_size=case["k"], padding=case["padding"], stride=stride, dilation=case["dilation"], groups=case["groups"]
    )
    want_w, want_b = [], []
    for i in range(x.shape[0]):
        conv.zero_grad()
        loss(mod(x[i : i + 1])).backward()
        want_w.append(conv.weight.grad.clone())
        want_b.append(conv.bias.grad.clone())
    torch.testing.assert_close(gs_w, torch.stack(want_w), rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(gs_b, torch.stack(want_b), rtol=1e-10, atol=1e-10)


def test_conv2d_empty_batch_has_batch_dim_one():
    gs_w, gs_b = O.conv2d_grad_sample(
        torch.zeros(0, 4, 5, 5), torch.zeros(0, 6, 5, 5), kernel_size=(3, 3), padding=(1, 1), stride=(1, 1), dilation=(1, 1), groups=2
    )
    assert gs_w.shape == (1, 6, 2, 3, 3) and gs_b.shape == (1, 6)
    assert gs_w.abs().sum() == 0


# ---- Embedding ------------------------------------------------------------------------
def test_embedding_grad_sample_vs_microbatch():
    torch.manual_seed(6)
    emb = nn.Embedding(9, 4, padding_idx=2).double()
    ids = torch.randint(0, 9, (5, 3, 2))
    ids[0, 0, 0] = 2  # padding_idx is not special-cased by the reference's sampler
    wts = torch.randn(5, 3, 2, 4, dtype=torch.float64)
    y = emb(ids)
    gs = O.embedding_grad_sample(ids, wts, 9)
    # closed form: gs[n, v] = sum of wts rows whose id is v
    want = torch.zeros(5, 9, 4, dtype=torch.float64)
    for n in range(5):
        for t, v in enumerate(ids[n].flatten().tolist()):
            want[n, v] += wts[n].reshape(-1, 4)[t]
    torch.testing.assert_close(gs, want, rtol=0, atol=1e-15)
    # autograd agrees away from padding_idx
    emb2 = nn.Embedding(9, 4).double()
    for n in range(5):
        emb2.zero_grad()
        (emb2(ids[n : n + 1]) * wts[n : n + 1]).sum().backward()
        torch.testing.assert_close(gs[n], emb2.weight.grad)
    assert y.shape == (5, 3, 2, 4)


def test_embedding_norm_golden_vectors(embedding_norm_cases):
    for c in embedding_norm_cases:
        r = O.embedding_norm_sample(c["ids"], c["backprops"])
        torch.testing.assert_close(r["result_sqrt"], c["expected"], atol=1e-4, rtol=1e-4, msg=c["name"])
        if c["intermediates"]:
            im = c["intermediates"]
            assert r["unique_paired_indices"].tolist() == im["unique_paired_indices"]
            assert r["new_index_positions"].tolist() == im["new_index_positions"]
            torch.testing.assert_close(r["summed_gradients"].flatten(), torch.tensor(im["summed_gradients"]), atol=1e-6, rtol=1e-6)
            torch.testing.assert_close(r["sqr_gradient_sum"], torch.tensor(im["sqr_gradient_sum"]), atol=1e-6, rtol=1e-6)
            torch.testing.assert_close(r["result"], torch.tensor(im["result"]), atol=1e-6, rtol=1e-6)


def test_embedding_norm_equals_norm_of_grad_sample():
    torch.manual_seed(7)
    ids = torch.randint(0, 6, (7, 10))  # many duplicates inside a sample
    b = torch.randn(7, 10, 5, dtype=torch.float64)
    gs = O.embedding_grad_sample(ids, b, 6)
    r = O.embedding_norm_sample(ids, b)
    torch.testing.assert_close(r["result_sqrt"], gs.flatten(1).norm(dim=1), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("mode", ["sum", "mean"])
def test_embedding_bag_grad_sample_vs_microbatch_and_repeat_rule(mode):
    """Bags without repeated indices: equal to batch-of-one autograd of nn.EmbeddingBag. A repeated
    index receives the backprop once (embedding.py:84-87 uses an indexed "+="): hand-computed."""
    torch.manual_seed(15)
    V, D = 9, 4
    bag = nn.EmbeddingBag(V, D, mode=mode).double()
    index = torch.tensor([1, 4, 7, 0, 2, 3, 5, 8, 6])
    offsets = torch.tensor([0, 3, 4, 8])  # bags of 3, 1, 4, 1
    out = bag(index, offsets)
    b = torch.autograd.grad((out.pow(2)).sum(), out)[0]
    gs = O.embedding_bag_grad_sample(index, offsets, b, V, mode)
    ends = [3, 4, 8, 9]
    for i in range(4):
        bag.zero_grad()
        lo, hi = int(offsets[i]), ends[i]
        o = bag(index[lo:hi], torch.tensor([0]))
        (o.pow(2)).sum().backward()
        torch.testing.assert_close(gs[i], bag.weight.grad, rtol=1e-12, atol=1e-12)
    # repeated index: the row is written once
    b2 = torch.tensor([[1.0, 2.0, 3.0, 4.0]], dtype=torch.float64)
    g2 = O.embedding_bag_grad_sample(torch.tensor([2, 2, 5]), torch.tensor([0]), b2, V, mode)
    want = b2[0] / (3 if mode == "mean" else 1)
    assert torch.equal(g2[0, 2], want) and torch.equal(g2[0, 5], want) and g2[0].abs().sum() == 2 * want.abs().sum()


CONV3D_CASES = [
    dict(C=2, O=3, k=(2, 3, 2), stride=(1, 1, 1), padding=(0, 1, 0), dilation=(1, 1, 1), groups=1, size=(4, 5, 6)),
    dict(C=4, O=4, k=(3, 2, 2), stride=(2, 1, 2), padding=(1, 0, 2), dilation=(1, 2, 1), groups=2, size=(6, 5, 7)),
    dict(C=2, O=2, k=(2, 2, 3), stride=(1, 1, 1), padding="same", dilation=(2, 1, 1), groups=1, size=(5, 4, 6)),
    dict(C=3, O=6, k=(1, 1, 1), stride=(1, 2, 1), padding="valid", dilation=(1, 1, 1), groups=3, size=(3, 4, 3)),
]


@pytest.mark.parametrize("case", CONV3D_CASES)
def test_conv3d_grad_sample_vs_microbatch(case):
    torch.manual_seed(16)
    conv = nn.Conv3d(case["C"], case["O"], case["k"], stride=case["stride"], padding=case["padding"],
                     dilation=case["dilation"], groups=case["groups"]).double()
    x = torch.randn(3, case["C"], *case["size"], dtype=torch.float64)
    loss = lambda y: y.pow(2).sum()  # noqa: E731
    b = _backprops(conv, x, loss)
    gs_w, gs_b = O.conv3d_grad_sample(x, b, kernel_size=case["k"], padding=case["padding"], stride=case["stride"],
                                      dilation=case["dilation"], groups=case["groups"])
    want = _per_sample_autograd(conv, x, loss)
    torch.testing.assert_close(gs_w, want["weight"], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(gs_b, want["bias"], rtol=1e-10, atol=1e-10)


def test_unfold3d_of_a_depth_one_volume_is_unfold2d():
    torch.manual_seed(17)
    x = torch.randn(2, 3, 6, 7, dtype=torch.float64)
    u2 = O.unfold2d(x, kernel_size=(3, 2), padding=(1, 2), stride=(2, 1), dilation=(1, 2))
    u3 = O.unfold3d(x.unsqueeze(2), kernel_size=(1, 3, 2), padding=(0, 1, 2), stride=(1, 2, 1), dilation=(1, 1, 2))
    assert torch.equal(u2, u3)


# ---- Norm layers ----------------------------------------------------------------------
def test_group_norm_grad_sample_vs_microbatch():
    torch.manual_seed(8)
    gn = nn.GroupNorm(2, 6, eps=1e-3).double()
    gn.weight.data.normal_()
    gn.bias.data.normal_()
    x = torch.randn(4, 6, 3, 5, dtype=torch.float64)
    loss = lambda y: y.pow(2).sum()  # noqa: E731
    b = _backprops(gn, x, loss)
    gs_w, gs_b = O.group_norm_grad_sample(x, b, 2, 1e-3)
    want = _per_sample_autograd(gn, x, loss)
    torch.testing.assert_close(gs_w, want["weight"], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(gs_b, want["bias"], rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("shape", [(4, 8), (3, 5, 8), (2, 3, 4, 8)])
def test_rms_norm_grad_sample_vs_microbatch(shape):
    torch.manual_seed(9)
    rn = nn.RMSNorm(8, eps=1e-5).double()
    rn.weight.data.normal_()
    x = torch.randn(*shape, dtype=torch.float64)
    loss = lambda y: y.pow(2).sum()  # noqa: E731
    b = _backprops(rn, x, loss)
    gs_w = O.rms_norm_grad_sample(x, b, (8,), 1e-5)
    want = _per_sample_autograd(rn, x, loss)
    torch.testing.assert_close(gs_w, want["weight"], rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("shape,normalized", [((4, 8), (8,)), ((3, 5, 8), (8,)), ((2, 3, 4, 6), (4, 6))])
def test_layer_norm_grad_sample_vs_microbatch(shape, normalized):
    torch.manual_seed(13)
    ln = nn.LayerNorm(normalized, eps=1e-4).double()
    ln.weight.data.normal_()
    ln.bias.data.normal_()
    x = torch.randn(*shape, dtype=torch.float64) * 2 + 1
    loss = lambda y: y.pow(3).sum()  # noqa: E731
    b = _backprops(ln, x, loss)
    gs_w, gs_b = O.layer_norm_grad_sample(x, b, normalized, 1e-4)
    want = _per_sample_autograd(ln, x, loss)
    torch.testing.assert_close(gs_w, want["weight"], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(gs_b, want["bias"], rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("cls,shape", [(nn.InstanceNorm1d, (3, 4, 7)), (nn.InstanceNorm2d, (2, 3, 4, 5))])
def test_instance_norm_grad_sample_vs_microbatch(cls, shape):
    torch.manual_seed(14)
    inorm = cls(shape[1], eps=1e-3, affine=True).double()
    inorm.weight.data.normal_()
    inorm.bias.data.normal_()
    x = torch.randn(*shape, dtype=torch.float64) + 0.5
    loss = lambda y: y.pow(2).sum()  # noqa: E731
    b = _backprops(inorm, x, loss)
    gs_w, gs_b = O.instance_norm_grad_sample(x, b, 1e-3)
    want = _per_sample_autograd(inorm, x, loss)
    torch.testing.assert_close(gs_w, want["weight"], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(gs_b, want["bias"], rtol=1e-10, atol=1e-10)
    # and it is group normalisation with one channel per group
    gw2, gb2 = O.group_norm_grad_sample(x, b, shape[1], 1e-3)
    torch.testing.assert_close(gs_w, gw2, rtol=1e-12, atol=1e-12)


# ---- Clipping -------------------------------------------------------------------------
def test_clip_and_accumulate_closed_form():
    torch.manual_seed(10)
    g1 = torch.randn(6, 3, 4, dtype=torch.float64)
    g2 = torch.randn(6, 5, dtype=torch.float64) * 0.01
    g1[0] *= 100  # one sample far above C, and
    g1[1] *= 1e-3  # one below it
    g2[1] *= 1e-3
    C = 0.7
    norms, clip, summed = O.clip_and_accumulate([g1, g2], C)
    want_norm = torch.sqrt(g1.flatten(1).pow(2).sum(1) + g2.pow(2).sum(1))
    torch.testing.assert_close(norms, want_norm)
    assert clip[1] == 1.0 and clip[0] < 1e-2
    for i in range(6):
        assert math.isclose(clip[i].item(), min(1.0, C / (want_norm[i].item() + 1e-6)), rel_tol=1e-12)
    torch.testing.assert_close(summed[0], sum(clip[i] * g1[i] for i in range(6)))
    torch.testing.assert_close(summed[1], sum(clip[i] * g2[i] for i in range(6)))
    # accumulation onto an earlier summed_grad
    _, _, again = O.clip_and_accumulate([g1, g2], C, summed=summed)
    torch.testing.assert_close(again[0], 2 * summed[0])


def test_clip_batch_of_one_has_norm_C():
    torch.manual_seed(11)
    g = [torch.randn(1, 10, 10), torch.randn(1, 7)]
    _, _, summed = O.clip_and_accumulate(g, 1.0)
    total = math.sqrt(sum(s.pow(2).sum().item() for s in summed))
    assert round(total, 3) == 1.0


def test_clip_empty_batch():
    norms, clip, summed = O.clip_and_accumulate([torch.zeros(0, 3, 2)], 1.0)
    assert clip.shape == (0,) and summed[0].shape == (3, 2) and summed[0].abs().sum() == 0


def test_per_layer_clipping_reduces_to_flat_clipping_and_bounds_every_layer():
    """What the mathematics fixes for perlayeroptimizer.py:58-76: with a single parameter it is flat
    clipping; with huge bounds the plain sum; with tiny bounds every parameter's clipped sample
    has norm C_k exactly, so a batch of one gives sums of norms C_k."""
    torch.manual_seed(12)
    g1, g2 = torch.randn(5, 3, 4, dtype=torch.float64), torch.randn(5, 6, dtype=torch.float64)
    _, _, flat = O.clip_and_accumulate([g1], 0.5)
    clips, summed = O.per_layer_clip_and_accumulate([g1], [0.5])
    torch.testing.assert_close(summed[0], flat[0])
    clips, summed = O.per_layer_clip_and_accumulate([g1, g2], [1e9, 1e9])
    assert all((c == 1).all() for c in clips)
    torch.testing.assert_close(summed[0], g1.sum(0))
    torch.testing.assert_close(summed[1], g2.sum(0))
    clips, summed = O.per_layer_clip_and_accumulate([g1[:1], g2[:1]], [0.3, 0.02])
    assert math.isclose(summed[0].norm().item(), 0.3, rel_tol=1e-5)
    assert math.isclose(summed[1].norm().item(), 0.02, rel_tol=1e-4)
    # the layers do not see each other: scaling one leaves the other's factors alone
    c_a, _ = O.per_layer_clip_and_accumulate([g1, g2], [0.5, 0.5])
    c_b, _ = O.per_layer_clip_and_accumulate([g1 * 100, g2], [0.5, 0.5])
    torch.testing.assert_close(c_a[1], c_b[1])


def test_adaclip_update_moves_towards_the_target_quantile():
    """adaclipoptimizer.py:119-121, 181-194 on hand-checked numbers."""
    clip = torch.tensor([1.0, 1.0, 0.5, 0.25])  # two of four unclipped
    count, new = O.adaclip_update(clip, 2.0, target_quantile=0.5, learning_rate=0.3, min_bound=0.1, max_bound=10.0)
    assert count == 2.0 and new == 2.0  # at the target: no change
    count, new = O.adaclip_update(clip, 2.0, 0.75, 0.3, 0.1, 10.0)
    assert math.isclose(new, 2.0 * math.exp(0.3 * 0.25))  # too few unclipped: the bound grows
    count, new = O.adaclip_update(torch.ones(4), 2.0, 0.5, 0.3, 0.1, 10.0)
    assert count == 4.0 and math.isclose(new, 2.0 * math.exp(-0.15))
    assert O.adaclip_update(torch.zeros(4), 9.0, 0.9, 5.0, 0.1, 10.0)[1] == 10.0
    assert O.adaclip_update(torch.ones(4), 0.11, 0.0, 5.0, 0.1, 10.0)[1] == 0.1


def test_clipping_coef_from_norm_samples():
    ns = [torch.tensor([3.0, 0.0, 0.3]), torch.tensor([4.0, 0.0, 0.4])]
    torch.testing.assert_close(O.per_sample_norm(ns), torch.tensor([5.0, 0.0, 0.5]))
    coef = O.clipping_coef(ns, 1.0)
    torch.testing.assert_close(coef, torch.tensor([1.0 / (5.0 + 1e-6), 1.0, 1.0]))


def test_noise_zero_std_is_exact_zero_and_does_not_touch_rng():
    g = torch.Generator().manual_seed(5)
    before = g.get_state().clone()
    z = O.generate_noise(0.0, torch.ones(3, 4), generator=g)
    assert z.abs().sum() == 0 and torch.equal(before, g.get_state())


def test_noise_statistics_and_scale():
    g = torch.Generator().manual_seed(6)
    z = O.generate_noise(2.5, torch.zeros(400_000), generator=g)
    assert abs(z.mean().item()) < 0.02 and abs(z.std().item() - 2.5) < 0.02
    zs = O.generate_noise(2.5, torch.zeros(400_000), generator=g, secure_mode=True)
    assert abs(zs.mean().item()) < 0.02 and abs(zs.std().item() - 2.5) < 0.02
    summed = [torch.full((4, 2), 8.0)]
    grads = O.add_noise_and_scale(summed, [torch.Size([2, 4])], 0.0, 1.0, 4, "mean", accumulated_iterations=2)
    assert grads[0].shape == (2, 4) and torch.all(grads[0] == 1.0)
    grads = O.add_noise_and_scale(summed, [torch.Size([2, 4])], 0.0, 1.0, 4, "sum")
    assert torch.all(grads[0] == 8.0)


def test_private_step_equals_plain_sgd_when_nothing_clips():
    """sigma = 0 and a huge C: clip-accumulate + scale reproduces autograd's mean gradient."""
    torch.manual_seed(12)
    lin = nn.Linear(6, 3)
    x = torch.randn(8, 6)
    y = torch.randint(0, 3, (8,))
    out = lin(x)
    out.retain_grad()
    F.cross_entropy(out, y).backward()
    b = O.scale_backprops(out.grad, 8, "mean")
    gs_w, gs_b = O.linear_grad_sample(x, b)
    _, clip, summed = O.clip_and_accumulate([gs_w, gs_b], 1e20)
    assert torch.all(clip == 1.0)
    grads = O.add_noise_and_scale(summed, [lin.weight.shape, lin.bias.shape], 0.0, 1e20, 8, "mean")
    torch.testing.assert_close(grads[0], lin.weight.grad, atol=1e-7, rtol=1e-3)
    torch.testing.assert_close(grads[1], lin.bias.grad, atol=1e-7, rtol=1e-3)


def test_store_grad_sample_pads_to_max_batch_len():
    gs = torch.ones(2, 3)
    buf = O.store_grad_sample(gs, 4)
    assert buf.shape == (4, 3) and buf[:2].sum() == 6 and buf[2:].abs().sum() == 0


# ---- Philox ---------------------------------------------------------------------------
def test_philox_known_answers():
    """Random123's kat_vectors for philox4x32-10."""
    kat = [
        ([0, 0, 0, 0], [0, 0], [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]),
        ([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2, [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]),
        (
            [0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344],
            [0xA4093822, 0x299F31D0],
            [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1],
        ),
    ]
    for ctr, key, want in kat:
        got = O.philox4x32_10(np.array(ctr, dtype=np.uint32), np.array(key, dtype=np.uint32))
        assert [int(v) for v in got] == want


def test_philox_normal_moments():
    z = O.philox_normal(1_000_000, seed=1234, offset=7)
    assert abs(z.mean()) < 5e-3 and abs(z.std() - 1.0) < 5e-3
    assert abs((z**3).mean()) < 2e-2 and abs((z**4).mean() - 3.0) < 5e-2
    z2 = O.philox_normal(1_000_000, seed=1234, offset=8)
    assert abs(np.corrcoef(z, z2)[0, 1]) < 5e-3


def test_ghost_adaptive_update_hand_numbers_and_identities():
    """adaptive_clipping_utils.py:123-175 by hand. norms (0.5, 1, 2, 4), C = 1: two of four are
    unclipped (<=), so at target 0.5 the bound is a fixed point; at target 0.75 it grows by
    exp(0.2 * 0.25)."""
    norms = torch.tensor([0.5, 1.0, 2.0, 4.0])
    new, sigma, coeff = O.ghost_adaptive_update(norms, 1.0, 0.5, 0.2, 0.1, 10.0, noise_multiplier=0.0)
    assert new == 1.0 and sigma == 0.0
    assert torch.equal(coeff, torch.tensor([1.0, 1.0, 0.5, 0.25]))
    new, _, coeff = O.ghost_adaptive_update(norms, 1.0, 0.75, 0.2, 0.1, 10.0, 0.0)
    assert new == pytest.approx(math.exp(0.05), rel=1e-12)
    # every clipped sample lands exactly on the new bound, unclipped ones are untouched
    scaled = coeff.double() * norms.double()
    assert torch.allclose(scaled[2:], torch.full((2,), new, dtype=torch.float64), rtol=1e-6)
    assert torch.equal(scaled[:2], norms[:2].double())
    # the count noise enters the fraction additively: +1 sample of noise at n = 4 is +0.25
    noisy, _, _ = O.ghost_adaptive_update(norms, 1.0, 0.5, 0.2, 0.1, 10.0, 0.0, count_noise=1.0)
    assert noisy == pytest.approx(math.exp(-0.2 * 0.25), rel=1e-12)
    # clamps
    assert O.ghost_adaptive_update(norms, 1.0, 1.0, 50.0, 0.1, 3.0, 0.0)[0] == 3.0
    assert O.ghost_adaptive_update(norms, 1.0, 0.0, 50.0, 0.4, 3.0, 0.0)[0] == 0.4
    # privacy composition of the two Gaussian mechanisms: sigma'^-2 + (2 n / 20)^-2 == sigma^-2
    big = torch.rand(200)
    _, sigma, _ = O.ghost_adaptive_update(big, 1.0, 0.5, 0.2, 0.1, 10.0, noise_multiplier=1.3)
    assert sigma > 1.3
    assert sigma ** -2 + (2 * 200 / 20.0) ** -2 == pytest.approx(1.3 ** -2, rel=1e-12)


def test_tied_embedding_norm_is_the_norm_of_autograds_shared_gradient():
    """A table used as nn.Embedding weight and as nn.Linear weight: with a batch of one,
    autograd's gradient of the shared parameter is the sample's whole gradient, so its norm
    pins the oracle; the decomposition into the two ghost norms and the cross term pins the
    inner product."""
    torch.manual_seed(12)
    V, D, n, T = 11, 6, 4, 5
    emb = nn.Embedding(V, D).double()
    ids = torch.randint(0, V, (n, T))
    ids[1, 1:4] = ids[1, 0]  # repeated ids in one sample
    mix = torch.randn(D, D).double()
    y = torch.randint(0, V, (n, T))
    e_rows, a_rows, g_rows, want = [], [], [], []
    for i in range(n):
        emb.zero_grad()
        h = emb(ids[i : i + 1])
        h.retain_grad()
        a = torch.tanh(h @ mix)
        a.retain_grad()
        logits = F.linear(a, emb.weight)
        logits.retain_grad()
        F.cross_entropy(logits.flatten(0, 1), y[i], reduction="sum").backward()
        want.append(emb.weight.grad.norm())
        e_rows.append(h.grad[0])
        a_rows.append(a.detach()[0])
        g_rows.append(logits.grad[0])
    e, a, g = torch.stack(e_rows), torch.stack(a_rows), torch.stack(g_rows)
    norm, cross = O.tied_embedding_norm_sample(ids, e, a, g)
    torch.testing.assert_close(norm, torch.stack(want), rtol=1e-12, atol=1e-14)
    n_emb = O.embedding_norm_sample(ids, e)["result_sqrt"]
    n_head, _ = O.linear_norm_sample(a, g, bias=False)
    torch.testing.assert_close(norm**2, n_emb**2 + n_head**2 + 2 * cross, rtol=1e-10, atol=1e-14)
    assert (cross.abs() > 1e-6).all()  # the term is not negligible in this setting
