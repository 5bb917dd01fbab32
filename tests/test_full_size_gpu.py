"""GPU parity at the full sizes of the five benchmark configurations.

The CPU oracle cannot recompute 8.6 GB of per-sample gradients or a 1024 x 1024 x 32000 Gram for
every sample in test time, so full-size runs are checked through what does not depend on the
size: closed forms that collapse to a small CPU computation (a clip-weighted sum of rank-one
gradients is one thin matrix product), the oracle on a few samples of the batch (every sample
is independent on this path), exact scaling by powers of two, invariance under a permutation of
the positions t, and additivity in the backprops. Tolerances are the stated bar: fp32 within
rel 1e-5 of the tensor's scale, bf16 inputs with fp32 accumulation within 2e-2 (in practice
1e-4, since the inputs are exact in bf16), integer-indexed outputs exact.
"""

import math

import pytest
import torch

from _compare import rel_err, rel_measures
from oracle import dp_oracle as O

pytestmark = pytest.mark.gpu

FP32_REL = 1e-5


@pytest.fixture(scope="module")
def K():
    from opacus_amd import kernels

    return kernels


def dev(t):
    return t.to("cuda")


# ---- C2: Linear 4096 x 4096, batch 128, T = 1, fp32 ----------------------------------------
def test_c2_linear_grad_sample_clip_accumulate_noise(K):
    n, d = 128, 4096
    torch.manual_seed(0)
    a, b = torch.randn(n, d), torch.randn(n, d)
    da, db = dev(a), dev(b)
    gs, sumsq = K.linear_grad_sample(db, da)
    assert gs.shape == (n, d, d)
    # rank-one structure: every entry is one fp32 product, so sampled entries are exact
    g = torch.Generator().manual_seed(1)
    ii, jj, kk = (torch.randint(0, hi, (4096,), generator=g) for hi in (n, d, d))
    got = gs[dev(ii), dev(jj), dev(kk)].cpu()
    assert torch.equal(got, b[ii, jj] * a[ii, kk])
    # a whole sample against the oracle's einsum
    want0, _ = O.linear_grad_sample(a[5:6], b[5:6])
    assert torch.equal(gs[5].cpu(), want0[0])
    # squared norms: closed form |b|^2 |a|^2 in float64
    want_ss = a.double().pow(2).sum(1) * b.double().pow(2).sum(1)
    assert rel_err(sumsq, want_ss) < FP32_REL
    # and the streaming norm kernel over the 8.6 GB tensor agrees with it
    assert rel_err(K.sumsq_rows([gs])[0], want_ss) < FP32_REL
    # clip-weighted sum = (clip * B)^T A, a thin product the CPU does in float64
    C = math.sqrt(want_ss.median().item())  # about half of the samples are clipped
    norm, clip = K.clip_factor(sumsq.reshape(1, -1), C)
    want_clip = (C / (want_ss.sqrt() + 1e-6)).clamp(max=1.0)
    assert rel_err(clip, want_clip) < FP32_REL and 0 < (want_clip < 1).sum() < n
    summed = torch.empty(d, d, device="cuda")
    K.clip_accumulate([gs], clip, [summed], accumulate=False)
    want_sum = (want_clip[:, None] * b.double()).t() @ a.double()
    assert rel_err(summed, want_sum) < FP32_REL
    K.clip_accumulate([gs], clip, [summed], accumulate=True)
    assert rel_err(summed, 2 * want_sum) < FP32_REL
    # noise at full size: exact when std = 0, N(0, std^2) / denom otherwise, repeatable
    grad = torch.empty_like(summed)
    K.add_noise(summed, grad, 0.0, 128.0, 3, 0)
    assert torch.equal(grad, summed / 128.0)
    K.add_noise(summed, grad, 2.0, 4.0, 3, 8)
    z = (grad.double() * 4.0 - summed.double()) / 2.0
    P = z.numel()
    assert abs(z.mean().item()) < 5 / math.sqrt(P) and abs(z.std().item() - 1.0) < 5 / math.sqrt(2 * P)
    again = torch.empty_like(grad)
    K.add_noise(summed, again, 2.0, 4.0, 3, 8)
    assert torch.equal(grad, again)


# ---- C3 / C5: ghost norms, bf16 ---------------------------------------------------------------
@pytest.mark.parametrize(
    "n,T,fin,fout,check",
    [
        (32, 512, 1024, 4096, 3),  # C3 fc1
        (32, 512, 4096, 1024, 3),  # C3 fc2
        (16, 1024, 2048, 2048, 2),  # C5 q / o
        (16, 1024, 2048, 512, 2),  # C5 k / v: thin enough for the direct route
        (16, 1024, 2048, 5632, 2),  # C5 gate / up
        (16, 1024, 5632, 2048, 2),  # C5 down
        (16, 1024, 2048, 32000, 1),  # C5 LM head
    ],
)
def test_ghost_norm_full_size(K, n, T, fin, fout, check):
    torch.manual_seed(T + fout)
    a = torch.randn(n, T, fin, device="cuda").bfloat16()
    b = (torch.randn(n, T, fout, device="cuda") * 0.02).bfloat16()
    nw, nb = K.linear_ghost_norm(b, a, want_weight=True, want_bias=True)
    assert nw.shape == (n,) and nw.dtype == torch.float32
    # the oracle (float64 Grams) on a few samples: samples are independent
    want_w, want_b = O.linear_norm_sample(a[:check].cpu().double(), b[:check].cpu().double())
    assert rel_err(nw[:check], want_w) < 1e-4 and rel_err(nb[:check], want_b) < 1e-4
    # the same samples alone give the same norms (other tiling of the launch)
    alone_w, alone_b = K.linear_ghost_norm(b[:check].contiguous(), a[:check].contiguous(), want_weight=True, want_bias=True)
    assert rel_err(alone_w, nw[:check]) < FP32_REL and rel_err(alone_b, nb[:check]) < FP32_REL
    # exact scaling: doubling the backprops doubles every accumulator exactly
    nw2, nb2 = K.linear_ghost_norm((b.float() * 2).bfloat16(), a, want_weight=True, want_bias=True)
    assert torch.equal(nw2, 2 * nw) and torch.equal(nb2, 2 * nb)
    # the scale argument is the same factor
    nw3, _ = K.linear_ghost_norm(b, a, scale=2.0, want_weight=True, want_bias=False)
    assert rel_err(nw3, 2 * nw) < 1e-6
    # invariance under a permutation of the positions t
    perm = torch.randperm(T, device="cuda")
    nwp, nbp = K.linear_ghost_norm(b[:, perm].contiguous(), a[:, perm].contiguous(), want_weight=True, want_bias=True)
    assert rel_err(nwp, nw) < FP32_REL and rel_err(nbp, nb) < FP32_REL
    # the norm of the bias gradient is |sum_t b_t| for every sample
    assert rel_err(nb, b.double().sum(1).norm(dim=1)) < 1e-4


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n,T,fin,fout", [(16, 1024, 2048, 1024), (8, 1000, 2048, 5632)])
def test_linear_grad_sample_with_sequence_full_size(K, dtype, n, T, fin, fout):
    """The materialising counterpart of the ghost norms at C5's layer shapes (hooks mode on a
    sequence model): per-sample weight gradients contracted over T by the direct-load kernels."""
    torch.manual_seed(T + fout)
    a = torch.randn(n, T, fin, device="cuda").to(dtype)
    b = (torch.randn(n, T, fout, device="cuda") * 0.02).to(dtype)
    gs, sumsq = K.linear_grad_sample(b, a)
    assert gs.shape == (n, fout, fin) and gs.dtype == dtype and sumsq.dtype == torch.float32
    tol = FP32_REL if dtype == torch.float32 else 2 ** -8  # one rounding to bf16 on the way out
    # the oracle (float64 einsum) on two samples: samples are independent
    want, _ = O.linear_grad_sample(a[:2].cpu().double(), b[:2].cpu().double())
    assert rel_err(gs[:2], want) < tol
    # the squared norms are those of the fp32 accumulators, before any rounding of gs
    assert rel_err(sumsq[:2], want.flatten(1).pow(2).sum(1)) < 1e-5
    # and they are the ghost norms of the same layer
    nw, _ = K.linear_ghost_norm(b, a, want_weight=True, want_bias=False)
    assert rel_err(sumsq.sqrt(), nw) < 1e-4
    # exact scaling: doubling the backprops doubles every accumulator exactly
    gs2, sumsq2 = K.linear_grad_sample((b.float() * 2).to(dtype), a)
    assert torch.equal(gs2.float(), 2 * gs.float()) and torch.equal(sumsq2, 4 * sumsq)
    # invariance under a permutation of the positions t (fp32 sums in another order)
    perm = torch.randperm(T, device="cuda")
    gsp, sumsqp = K.linear_grad_sample(b[:, perm].contiguous(), a[:, perm].contiguous())
    assert rel_err(gsp, gs) < (FP32_REL if dtype == torch.float32 else 2 ** -7) and rel_err(sumsqp, sumsq) < FP32_REL
    # additivity in the backprops, in fp32 outputs so that no rounding to bf16 interferes
    h = T // 2
    g1, _ = K.linear_grad_sample(b[:, :h].contiguous(), a[:, :h].contiguous(), out_dtype=torch.float32)
    g2, _ = K.linear_grad_sample(b[:, h:].contiguous(), a[:, h:].contiguous(), out_dtype=torch.float32)
    gf, _ = K.linear_grad_sample(b, a, out_dtype=torch.float32)
    assert rel_err(g1 + g2, gf) < FP32_REL


# ---- C4: Conv2d 64 -> 64, 3 x 3, 32 x 32 images, batch 256, fp32 ------------------------------
@pytest.mark.parametrize("pooled", [False, True])
def test_weighted_sum_past_32_bit_offsets(K, pooled):
    """n*T*out = 2.7e9 elements (5.4 GB of backprops): element and byte offsets inside the operand
    pass 2^31 and 2^32. Slices of the result against torch on the weighted operand in fp32, and
    linearity in the coefficients (scaling them by 4 scales the sum by 4, exactly)."""
    torch.manual_seed(13)
    n, T, fin, fout = 16, 4096, 256, 40960
    a = torch.randn(n, T, fin, device="cuda").bfloat16()
    b = torch.empty(n, T, fout, device="cuda", dtype=torch.bfloat16)
    for s in range(n):  # filled sample by sample: no fp32 copy of the whole tensor
        b[s] = (torch.randn(T, fout, device="cuda") * 0.05).bfloat16()
    c = torch.rand(n, device="cuda") * 0.9 + 0.1

    def run(coef):
        if pooled:
            return K.linear_weighted_sum_multi([(b, a, coef, 1.0)], out_dtype=torch.float32, pooled=True)[0]
        return K.linear_weighted_sum(b, a, coef, out_dtype=torch.float32)

    got = run(c)
    assert got.shape == (fout, fin)
    wa = (a.float() * c.view(n, 1, 1)).reshape(n * T, fin)
    for lo in (0, 20000, fout - 512):  # first, middle and last rows of the result
        want = b[:, :, lo : lo + 512].reshape(n * T, 512).float().t() @ wa
        assert rel_err(got[lo : lo + 512], want) < 1e-4, lo
    assert torch.equal(run(c * 4), got * 4)


def test_c4_conv_and_group_norm_full_size(K):
    n = 256
    torch.manual_seed(4)
    x, b = torch.randn(n, 64, 32, 32), torch.randn(n, 64, 32, 32)
    dx, db = dev(x), dev(b)
    geo = dict(kernel_size=(3, 3), stride=(1, 1), padding=(1, 1, 1, 1), dilation=(1, 1), groups=1)
    gs, sumsq = K.conv2d_grad_sample(dx, db, **geo)
    pick = [0, 17, 255]
    want, want_bias = O.conv2d_grad_sample(
        x[pick].double(), b[pick].double(), kernel_size=(3, 3), padding=(1, 1), stride=(1, 1), dilation=(1, 1), groups=1
    )
    assert rel_err(gs[pick], want) < FP32_REL
    assert rel_err(sumsq, gs.double().flatten(1).pow(2).sum(1)) < FP32_REL
    assert rel_err(K.conv_bias_grad_sample(db)[pick], want_bias) < FP32_REL
    # additivity in the backprops over the whole batch
    b2 = torch.randn(n, 64, 32, 32, device="cuda")
    gs2, _ = K.conv2d_grad_sample(dx, b2, **geo)
    gs12, _ = K.conv2d_grad_sample(dx, db + b2, **geo)
    assert rel_err(gs12, gs.double() + gs2.double()) < FP32_REL
    # GroupNorm(32, 64) on the same activations
    gw, gb = K.group_norm_grad_sample(dx, db, 32, 1e-5)
    want_w, want_b = O.group_norm_grad_sample(x.double(), b.double(), 32, 1e-5)
    assert rel_err(gw, want_w) < FP32_REL and rel_err(gb, want_b) < FP32_REL


@pytest.mark.parametrize(
    "n,C,Oc,H",
    [(256, 64, 64, 32), (64, 128, 128, 28), (32, 64, 64, 56)],  # C4's shape; 128-row blocks, runs of 4; a patch above 64 KB
)
def test_conv_bf16_kernel_against_the_fp32_kernel_full_size(K, n, C, Oc, H):
    """bf16 input runs its own kernel (bf16 MFMA). On the same bf16-exact data the fp32 kernel forms
    the same exact products and also accumulates in fp32, so the two must agree to fp32 rounding."""
    torch.manual_seed(n + H)
    x = torch.randn(n, C, H, H, device="cuda").bfloat16()
    b = torch.randn(n, Oc, H, H, device="cuda").bfloat16()
    geo = dict(kernel_size=(3, 3), stride=(1, 1), padding=(1, 1, 1, 1), dilation=(1, 1), groups=1)
    g16, s16 = K.conv2d_grad_sample(x, b, out_dtype=torch.float32, **geo)
    g32, s32 = K.conv2d_grad_sample(x.float(), b.float(), **geo)
    assert rel_err(g16, g32) < FP32_REL
    assert rel_err(s16, s32) < FP32_REL
    pick = [0, n - 1]
    want, _ = O.conv2d_grad_sample(
        x[pick].cpu().double(), b[pick].cpu().double(), kernel_size=(3, 3), padding=(1, 1), stride=(1, 1), dilation=(1, 1), groups=1
    )
    assert rel_err(g16[pick], want) < FP32_REL


# ---- C5: Embedding ghost norm and RMSNorm at batch 16, seq 1024, dim 2048, bf16 ---------------
def test_c5_embedding_and_rms_norm_full_size(K):
    n, T, D, V = 16, 1024, 2048, 32000
    torch.manual_seed(5)
    ids = torch.randint(0, V, (n, T))
    ids[3, :500] = ids[3, 0]  # one sample full of repeats
    b = (torch.randn(n, T, D) * 0.02).bfloat16()
    x = torch.randn(n, T, D).bfloat16()
    got = K.embedding_ghost_norm(dev(ids), dev(b))
    want = O.embedding_norm_sample(ids, b.double())["result_sqrt"]
    assert rel_err(got, want) < 1e-4
    # the integer stage is exact at full size too
    uniq, inverse = O.embedding_unique_pairs(ids)
    g_uniq, g_inv = K.embedding_unique_pairs(dev(ids))
    assert torch.equal(g_uniq.cpu(), uniq) and torch.equal(g_inv.cpu(), inverse)
    gw = K.rms_norm_grad_sample(dev(x), dev(b), D, 1e-5)
    want_w = O.rms_norm_grad_sample(x.double(), b.double(), (D,), 1e-5)
    assert rel_err(gw, want_w) < 2e-2  # the output is rounded to bf16
    gw32 = K.rms_norm_grad_sample(dev(x.float()), dev(b.float()), D, 1e-5)
    assert rel_err(gw32, want_w) < FP32_REL


# ---- C5 with tied embeddings: the cross term at batch 16, seq 1024, dim 2048, vocab 32000 ----------
def test_c5_tied_embedding_cross_term_full_size(K):
    n, T, D, V = 16, 1024, 2048, 32000
    torch.manual_seed(6)
    ids = torch.randint(0, V, (n, T), device="cuda")
    ids[2, :300] = ids[2, 0]
    e = (torch.randn(n, T, D, device="cuda") * 0.02).bfloat16()
    a = torch.randn(n, T, D, device="cuda").bfloat16()
    g = (torch.randn(n, T, V, device="cuda") * 0.01).bfloat16()
    got = K.tied_embedding_cross_term(ids, e, a, g)
    # the definition in float64, sample by sample (plain torch: an independent route)
    want = []
    for i in range(n):
        gathered = g[i].double().gather(1, ids[i].unsqueeze(0).expand(T, T))  # [t2, t] = g[t2, ids[t]]
        want.append((e[i].double() * (gathered.t() @ a[i].double())).sum())
    want = torch.stack(want)
    # the sum has ~2 M terms of either sign: compare on the scale of its terms' root sum of squares
    scale = (e.double().pow(2).sum((1, 2)) * a.double().pow(2).sum((1, 2)) / D).sqrt() * 0.01
    assert ((got.double() - want).abs() / scale).max().item() < 1e-4
    # exact scaling by a power of two, and invariance under a permutation of the embedding positions
    assert torch.equal(K.tied_embedding_cross_term(ids, (e.float() * 2).bfloat16(), a, g), 2 * got)
    perm = torch.randperm(T, device="cuda")
    gotp = K.tied_embedding_cross_term(ids[:, perm].contiguous(), e[:, perm].contiguous(), a, g)
    assert ((gotp - got).abs().double() / scale).max().item() < 1e-4
    # the oracle (materialised gradients) on one sample of the batch
    _, want0 = O.tied_embedding_norm_sample(ids[:1].cpu(), e[:1].cpu().float(), a[:1].cpu().float(), g[:1].cpu().float())
    assert abs(got[0].item() - want0.item()) / scale[0].item() < 1e-3


# ---- C1: the small CNN at batch 256, whole step against the oracle ------------------------------
def test_c1_small_cnn_full_batch_step():
    import copy

    import torch.nn.functional as F

    import bench
    import opacus_amd as A

    torch.manual_seed(0)
    net = bench.SmallCNN()
    n = 256
    x, y = torch.randn(n, 1, 28, 28), torch.randint(0, 10, (n,))
    names = [k for k, _ in net.named_parameters()]
    per_sample = {k: [] for k in names}
    for i in range(n):
        net.zero_grad()
        F.cross_entropy(net(x[i : i + 1]), y[i : i + 1], reduction="sum").backward()
        for k, p in net.named_parameters():
            per_sample[k].append(p.grad.clone())
    net.zero_grad()
    gs = [torch.stack(per_sample[k]) for k in names]
    norms, clip, summed = O.clip_and_accumulate(gs, 1.0)
    gsm = A.GradSampleModule(copy.deepcopy(net).cuda(), loss_reduction="mean")
    opt = A.DPOptimizer(torch.optim.SGD(gsm.parameters(), lr=0.1), noise_multiplier=0.0, max_grad_norm=1.0, expected_batch_size=n)
    opt.zero_grad()
    F.cross_entropy(gsm(x.cuda()), y.cuda()).backward()
    for (k, p), g in zip(gsm._module.named_parameters(), gs):
        assert rel_err(p.grad_sample, g) < 2e-5, k
    opt.step()
    for (k, p), s in zip(gsm._module.named_parameters(), summed):
        assert rel_err(p.grad, s / n) < 2e-5, k


# ---- Whole steps through the drop-in API at the configurations' full sizes, sigma = 0 ----------
# (the pattern of opacus/tests/grad_sample_module_fast_gradient_clipping_test.py:129-280 and
#  privacy_engine_test.py:220-273: per-sample norms, then the gradient the optimizer leaves in
#  p.grad, against an independent computation)
def _batch_of_one_grads(net, inputs, loss_of_one, n):
    """CPU autograd on one sample at a time (the reference's microbatch method,
    opacus/utils/per_sample_gradients_utils.py:96-167): per parameter, [n, *shape]."""
    out = [[] for _ in net.parameters()]
    for i in range(n):
        net.zero_grad(set_to_none=True)
        loss_of_one(net, inputs, i).backward()
        for k, p in enumerate(net.parameters()):
            out[k].append(p.grad.clone())
    net.zero_grad(set_to_none=True)
    return [torch.stack(g) for g in out]


def test_c2_whole_step_against_the_closed_form():
    """Linear 4096 -> 4096 with bias, batch 128: the clipped sum is (clip * B)^T A in closed form."""
    import opacus_amd as A

    n, d, C, lr = 128, 4096, 1.0, 0.05
    torch.manual_seed(2)
    lin = torch.nn.Linear(d, d)
    w0, b0 = lin.weight.detach().double().clone(), lin.bias.detach().double().clone()
    x, bp = torch.randn(n, d), torch.randn(n, d)
    gsm = A.GradSampleModule(lin.cuda(), loss_reduction="sum")
    opt = A.DPOptimizer(torch.optim.SGD(gsm.parameters(), lr=lr), noise_multiplier=0.0, max_grad_norm=C,
                        expected_batch_size=n, loss_reduction="sum")
    opt.zero_grad()
    gsm(x.cuda()).backward(bp.cuda())
    opt.step()
    xd, bd = x.double(), bp.double()
    norms = (bd.pow(2).sum(1) * xd.pow(2).sum(1) + bd.pow(2).sum(1)).sqrt()  # weight and bias together
    clip = (C / (norms + 1e-6)).clamp(max=1.0)
    want_w, want_b = (clip[:, None] * bd).t() @ xd, (clip[:, None] * bd).sum(0)
    assert rel_err(lin.weight.grad, want_w) < FP32_REL and rel_err(lin.bias.grad, want_b) < FP32_REL
    # weights after the step (privacy_engine_test.py:261-273 compares these)
    assert rel_err(lin.weight.detach(), w0 - lr * want_w) < 1e-6 and rel_err(lin.bias.detach(), b0 - lr * want_b) < 1e-6


def test_c4_whole_step_against_batch_of_one_autograd():
    """The ResNet block at batch 256 in hooks mode, the whole batch, two independent references.

    (a) CPU autograd on one sample at a time. Its ReLUs see pre-activations that differ from the
    GPU's in the last bits (other summation orders in the convolutions), and of the 33 M of them a
    few lie so close to zero that the two devices disagree on the sign: that sample's backprops
    then differ in one position, which is a per-cent change of one row of its gradients and has
    nothing to do with the samplers. So: all but a few samples within 2e-5, the few within 0.5.
    (b) The oracle's samplers (float64) on the activations and backprops that plain torch autograd
    produces on the GPU for the same batch: no ReLU can flip between the two, so every sample of
    every parameter is held to the bar, and so is the clipped mean gradient."""
    import copy

    import torch.nn.functional as F

    import bench
    import opacus_amd as A

    n = 256
    torch.manual_seed(4)
    net = bench.ResBlock()
    x, y = torch.randn(n, 64, 32, 32), torch.randint(0, 10, (n,))
    gsm = A.GradSampleModule(copy.deepcopy(net).cuda(), loss_reduction="mean")
    opt = A.DPOptimizer(torch.optim.SGD(gsm.parameters(), lr=0.1), noise_multiplier=0.0, max_grad_norm=1.0, expected_batch_size=n)
    opt.zero_grad()
    F.cross_entropy(gsm(x.cuda()), y.cuda()).backward()
    names = [k for k, _ in net.named_parameters()]
    got = [p.grad_sample.detach().cpu() for p in gsm._module.parameters()]

    # (a)
    gs = _batch_of_one_grads(net, (x, y), lambda m, xy, i: F.cross_entropy(m(xy[0][i : i + 1]), xy[1][i : i + 1], reduction="sum"), n)
    flipped = set()
    for k, g, w in zip(names, got, gs):
        assert g.shape == w.shape, k
        per_sample = torch.tensor([rel_err(g[i : i + 1], w[i : i + 1]) for i in range(n)])
        assert (per_sample < 0.5).all(), k
        flipped |= set(torch.nonzero(per_sample >= 2e-5).flatten().tolist())
    assert len(flipped) <= 8, sorted(flipped)

    # (b)
    plain = copy.deepcopy(net).cuda()
    store, handles = bench._cpu_capture(plain)
    F.cross_entropy(plain(x.cuda()), y.cuda()).backward()
    for h in handles:
        h.remove()
    want = []
    for m, (a, b) in store.items():
        want += bench._cpu_grad_samples(O, m, a.cpu().double(), b.cpu().double() * n)
    assert len(want) == len(got)
    for k, g, w in zip(names, got, want):
        assert rel_err(g, w) < FP32_REL, k
    _, _, summed = O.clip_and_accumulate(want, 1.0)
    opt.step()
    for k, p, sg in zip(names, gsm._module.parameters(), summed):
        assert rel_err(p.grad, sg / n) < FP32_REL, k


def _ghost_step(A, net, inputs, loss_call, n, C, single=False):
    gsm = A.GradSampleModuleFastGradientClipping(net, loss_reduction="mean", max_grad_norm=C, single_backward=single)
    opt = A.optimizers.DPOptimizerFastGradientClipping(
        torch.optim.SGD(gsm.parameters(), lr=0.01), noise_multiplier=0.0, max_grad_norm=C, expected_batch_size=n
    )
    opt.zero_grad()
    loss_call(gsm, opt, inputs).backward()
    norms = gsm.per_sample_gradient_norms.detach().clone()
    opt.pre_step()
    grads = [p.grad.detach().clone() for p in gsm._module.parameters()]
    gsm.to_standard_module()
    return norms, grads


def _bf16_bar(got, want, bar=2e-2):
    """bf16 models: the chain of bf16 roundings in forward and backward (ours and torch's) differs
    between devices, so whole-step results are held to the bf16 bar at tensor and sample scale."""
    t, s, _ = rel_measures(got, want)
    return max(t, s) < bar, (t, s)


def test_c3_whole_step_against_batch_of_one_autograd():
    """The MLP of config 3 (bf16, batch 32, T = 512) under ghost clipping: per-sample norms and the
    clipped mean gradient against CPU batch-of-one autograd in fp32 on the same (bf16) weights."""
    import copy

    import bench
    import opacus_amd as A

    n, T, C = 32, 512, 1.0
    torch.manual_seed(3)
    net = torch.nn.Sequential(torch.nn.Linear(1024, 4096), torch.nn.GELU(), torch.nn.Linear(4096, 1024)).bfloat16()
    x = torch.randn(n, T, 1024).bfloat16()
    ref = copy.deepcopy(net).float()
    gs = _batch_of_one_grads(ref, x.float(), lambda m, xx, i: m(xx[i : i + 1]).pow(2).flatten(1).mean(1).sum(), n)
    want_norms, clip, summed = O.clip_and_accumulate(gs, C)
    crit = {}

    def loss_call(model, opt, xx):
        crit["c"] = A.DPLossFastGradientClipping(model, opt, bench.PerSampleMSE("mean"), "mean")
        return crit["c"](model(xx), None)

    for single in (False, True):
        norms, grads = _ghost_step(A, copy.deepcopy(net).cuda(), x.cuda(), loss_call, n, C, single=single)
        ok, m = _bf16_bar(norms, want_norms)
        assert ok, ("norms", single, m)
        for k, (g, sg) in enumerate(zip(grads, summed)):
            ok, m = _bf16_bar(g, sg / n)
            assert ok, ("grad", k, single, m)


def test_c5_whole_step_norms_and_clipped_gradient():
    """The 4-layer decoder of config 5 (bf16, batch 16, seq 1024) under ghost clipping. Every
    sample's norm is checked against batch-of-one autograd in fp32 on a copy of the model (the
    reference's microbatch method, opacus/utils/per_sample_gradients_utils.py:96-167, as its own
    ghost-clipping test compares every sample,
    opacus/tests/grad_sample_module_fast_gradient_clipping_test.py:129-200): on the GPU with torch's
    own kernels for all 16, and on the CPU (~10 s a sample) for two of them. Samples are
    independent (a sub-batch gives the same norms, a permuted batch the permuted norms), and the
    gradient the step leaves is the gradient of sum_n coef[n] loss[n] / n, which plain autograd on a
    copy of the model computes."""
    import copy

    import torch.nn.functional as F

    import bench
    import opacus_amd as A

    n, T, V, C = 16, 1024, 32000, 1.0
    torch.manual_seed(5)
    net = bench.Llama().bfloat16()
    ids = torch.randint(0, V, (n, T))
    crit = {}

    def loss_call(model, opt, idx):
        m = idx.shape[0]
        crit["c"] = A.DPLossFastGradientClipping(model, opt, torch.nn.CrossEntropyLoss(), "mean")
        logits = model(idx)[:, :-1]
        return crit["c"](logits.reshape(-1, V).float(), idx[:, 1:].reshape(-1), shape=(m, T - 1, V))

    def loss_per_sample(model, idx):
        m = idx.shape[0]
        tok = F.cross_entropy(model(idx)[:, :-1].reshape(-1, V).float(), idx[:, 1:].reshape(-1), reduction="none")
        return tok.view(m, T - 1).mean(1)

    dids = ids.cuda()
    norms, grads = _ghost_step(A, copy.deepcopy(net).cuda(), dids, loss_call, n, C)
    assert norms.shape == (n,) and torch.isfinite(norms).all()
    # (1) two samples against CPU autograd in fp32 on the same weights
    ref = copy.deepcopy(net).float()
    for i in (0, 9):
        ref.zero_grad(set_to_none=True)
        loss_per_sample(ref, ids[i : i + 1]).sum().backward()
        want = torch.cat([p.grad.flatten() for p in ref.parameters()]).double().norm()
        assert abs(norms[i].item() - want.item()) / want.item() < 2e-2, (i, norms[i].item(), want.item())
    # (1b) all sixteen against the same computation on the GPU (fp32 weights, one sample at a time)
    ref = ref.cuda()
    want_all = []
    for i in range(n):
        ref.zero_grad(set_to_none=True)
        loss_per_sample(ref, dids[i : i + 1]).sum().backward()
        want_all.append(torch.sqrt(sum(p.grad.double().pow(2).sum() for p in ref.parameters())))
    want_all = torch.stack(want_all)
    worst = ((norms.double() - want_all).abs() / want_all).max().item()
    assert worst < 2e-2, (worst, norms.tolist(), want_all.tolist())
    del ref
    # (2) samples are independent: half the batch alone, and the batch in another order
    sub, _ = _ghost_step(A, copy.deepcopy(net).cuda(), dids[8:].contiguous(), loss_call, n // 2, C)
    assert rel_err(sub, norms[8:]) < 2e-3
    perm = torch.randperm(n)
    pn, _ = _ghost_step(A, copy.deepcopy(net).cuda(), dids[perm.cuda()].contiguous(), loss_call, n, C)
    assert rel_err(pn, norms[perm.cuda()]) < 2e-3
    # (3) the clipped mean gradient: plain autograd of sum_n coef[n] loss[n] / n on a copy
    coef = (C / (norms + 1e-6)).clamp(max=1.0)
    plain = copy.deepcopy(net).cuda()
    (coef * loss_per_sample(plain, dids)).sum().div(n).backward()
    for (k, p), g in zip(plain.named_parameters(), grads):
        ok, m = _bf16_bar(g, p.grad)
        assert ok, (k, m)
    # (4) with the second backward pass replaced by the contraction over the kept backprops
    _, grads1 = _ghost_step(A, copy.deepcopy(net).cuda(), dids, loss_call, n, C, single=True)
    # The embedding table against an fp32 computation of the same clipped sum: the (bf16) gradients
    # that reach the embedding's output in a plain pass of the mean loss, weighted per sample and
    # added per id in fp32. torch's own bf16 embedding backward, which (3) compared with, rounds
    # after every addition to a row that several tokens name; this is the sum before any rounding.
    seen = []
    weighted_grads = {k: p.grad.detach().clone() for k, p in plain.named_parameters()}
    plain.zero_grad(set_to_none=True)
    def watch_output(_module, _inputs, out):
        out.register_hook(lambda g: seen.append(g.detach()))  # (a forward hook's return value would replace the output)

    h = plain.emb.register_forward_hook(watch_output)
    loss_per_sample(plain, dids).mean().backward()
    h.remove()
    (bp,) = seen
    want_emb = torch.zeros(V, bp.shape[-1], device="cuda", dtype=torch.float32)
    want_emb.index_add_(0, dids.reshape(-1), (coef.float().view(n, 1, 1) * bp.float()).flatten(0, 1))
    for (k, _p), g in zip(plain.named_parameters(), grads1):
        if k == "emb.weight":
            # rows as the "samples" of the comparison: every table row is held to its own size
            t, row, _ = rel_measures(g, want_emb)
            assert max(t, row) < 2e-2, (k, "single, against the fp32 sum", t, row)
            continue
        ok, m = _bf16_bar(g, weighted_grads[k])
        assert ok, (k, "single", m)
