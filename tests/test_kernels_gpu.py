"""GPU parity: every HIP kernel, called through the C ABI, against the CPU oracle.

Tolerances follow the stated bar: fp32 within rel 1e-5, bf16 within rel 2e-2 with fp32
accumulation - each applied at tensor, sample and element scale (see _compare.py) - and
integer outputs bit-exact.
"""

import math

import numpy as np
import pytest
import torch

from _compare import assert_rel
from oracle import dp_oracle as O

pytestmark = pytest.mark.gpu

FP32_REL = 1e-5
BF16_REL = 2e-2


@pytest.fixture(scope="module")
def K():
    from opacus_amd import kernels

    return kernels


def dev(t):
    return t.to("cuda")


# ---- Linear per-sample gradients ---------------------------------------------------------
LINEAR_SHAPES = [
    # (n, middle dims, in, out)
    (4, (), 8, 4),  # T = 1, tiny
    (3, (), 130, 67),  # T = 1, odd sizes -> scalar path
    (16, (), 512, 32),  # C1 fc1 shape
    (5, (1,), 256, 96),  # 3-d with T = 1
    (3, (7,), 64, 64),  # MFMA 64x64 tiles, K smaller than one k tile
    (2, (50,), 200, 136),  # MFMA 128 tiles with ragged edges
    (2, (33,), 70, 30),  # MFMA small tile, odd sizes -> scalar loads
    (2, (4, 9), 132, 260),  # two middle dims
    (1, (300,), 128, 128),  # long K
    (2, (16,), 128, 128),  # exactly one k tile of the direct-load fp32 kernel
    (1, (17,), 68, 132),  # its last k tile repeats 15 rows of the first; sizes that are multiples of 4 only
    (2, (48,), 516, 260),  # three whole k tiles, ragged block tiles in both directions
]


@pytest.mark.parametrize("n,mid,fin,fout", LINEAR_SHAPES)
@pytest.mark.parametrize("scale", [1.0, 3.0])
def test_linear_grad_sample_f32(K, n, mid, fin, fout, scale):
    torch.manual_seed(n * 1000 + fin)
    a = torch.randn(n, *mid, fin)
    b = torch.randn(n, *mid, fout)
    want_w, want_b = O.linear_grad_sample(a, b * scale)
    gs, sumsq = K.linear_grad_sample(dev(b), dev(a), scale=scale)
    gb = K.linear_bias_grad_sample(dev(b), scale=scale)
    assert_rel(gs, want_w, FP32_REL, "weight")
    assert_rel(gb, want_b, FP32_REL, "bias")
    assert_rel(sumsq, want_w.double().flatten(1).pow(2).sum(1), 2e-5, "sumsq")
    gs16, _ = K.linear_grad_sample(dev(b), dev(a), scale=scale, out_dtype=torch.bfloat16)
    assert gs16.dtype == torch.bfloat16
    assert_rel(gs16, want_w, BF16_REL, "weight, fp32 in, bf16 out")


@pytest.mark.parametrize(
    "n,mid,fin,fout",
    [
        (4, (), 64, 32),
        (2, (40,), 136, 200),  # 128 tiles with ragged edges, K under one k tile
        (3, (5,), 30, 18),  # odd sizes: element-wise loads
        (2, (200,), 256, 384),  # whole 128 tiles, K = 3 k tiles + 8
        (3, (65,), 64, 72),  # 64 tiles, K = one k tile + 1
        (1, (7, 19), 132, 260),  # two middle dimensions, sizes that are multiples of 4 only
        (2, (128,), 1024, 8),  # a narrow output
        (2, (32,), 128, 128),  # exactly one k tile of the transposing-read kernel, one block tile
        (1, (33,), 72, 136),  # its last k tile repeats 31 rows of the first
        (2, (96,), 520, 264),  # three whole k tiles, ragged block tiles in both directions
        (1, (1000,), 128, 256),  # a long contraction: the ring wraps many times
        (3, (4, 16), 256, 128),  # 64 positions in two middle dimensions
    ],
)
@pytest.mark.parametrize("tile", [0, 128, 256])
def test_linear_grad_sample_bf16(K, n, mid, fin, fout, tile):
    """`tile` forces the 128 x 128 or the 256 x 256 variant of the transposing-read kernel where
    the shape qualifies for it (0: the library's own choice)."""
    torch.manual_seed(7)
    a = torch.randn(n, *mid, fin).bfloat16()
    b = torch.randn(n, *mid, fout).bfloat16()
    want_w, want_b = O.linear_grad_sample(a.float(), b.float())
    gs, sumsq = K.linear_grad_sample(dev(b), dev(a), tile=tile)
    assert gs.dtype == torch.bfloat16
    assert_rel(gs, want_w, BF16_REL, "weight bf16")
    assert_rel(K.linear_bias_grad_sample(dev(b)), want_b, BF16_REL, "bias bf16")
    assert_rel(sumsq, want_w.double().flatten(1).pow(2).sum(1), 1e-4, "sumsq (fp32 accumulators)")
    gs32, _ = K.linear_grad_sample(dev(b), dev(a), out_dtype=torch.float32, tile=tile)
    assert_rel(gs32, want_w, FP32_REL, "weight bf16 in, fp32 out")


def test_linear_grad_sample_mixed_activation_dtype_and_views(K):
    torch.manual_seed(8)
    a = torch.randn(6, 5, 40)
    b = torch.randn(5, 6, 24).transpose(0, 1)  # not contiguous
    want_w, _ = O.linear_grad_sample(a, b)
    gs, _ = K.linear_grad_sample(dev(b), dev(a).double())  # activations are cast to backprops' dtype
    assert_rel(gs, want_w, FP32_REL)


def test_linear_empty_batch(K):
    gs, sumsq = K.linear_grad_sample(torch.zeros(0, 4, device="cuda"), torch.zeros(0, 6, device="cuda"))
    assert gs.shape == (0, 4, 6) and sumsq.shape == (0,)


def test_linear_is_deterministic(K):
    torch.manual_seed(9)
    a, b = dev(torch.randn(8, 33, 200)), dev(torch.randn(8, 33, 136))
    g1, s1 = K.linear_grad_sample(b, a)
    g2, s2 = K.linear_grad_sample(b, a)
    assert torch.equal(g1, g2) and torch.equal(s1, s2)


# ---- Optimizer kernels ---------------------------------------------------------------
GS_SETS = [
    [(5, (3, 4)), (5, (7,))],  # tiny, odd -> scalar path
    [(64, (32, 512)), (64, (32,)), (64, (10, 32)), (64, (10,))],  # C1-like tail
    [(9, (40000,))],  # several chunks per row
    [(130, (16, 1, 8, 8)), (130, (16,))],  # n not a multiple of the unroll, row split
]


@pytest.mark.parametrize("spec", GS_SETS)
@pytest.mark.parametrize("C", [0.5, 1e20])
def test_clip_and_accumulate_f32(K, spec, C):
    torch.manual_seed(len(spec))
    gs = [torch.randn(n, *shape) * (0.01 if i % 2 else 1.0) for i, (n, shape) in enumerate(spec)]
    gs[0][0] *= 50.0
    norms, clip, summed = O.clip_and_accumulate(gs, C)
    dgs = [dev(g) for g in gs]
    ss = K.sumsq_rows(dgs)
    want_ss = torch.stack([g.double().flatten(1).pow(2).sum(1) for g in gs])
    assert_rel(ss, want_ss, FP32_REL, "sumsq")
    gnorm, gclip = K.clip_factor(ss, C)
    assert_rel(gnorm, norms, FP32_REL, "norm")
    assert_rel(gclip, clip, FP32_REL, "clip")
    outs = [torch.full(g.shape[1:], 7.0, device="cuda") for g in gs]
    K.clip_accumulate(dgs, gclip, outs, accumulate=False)
    for o, s in zip(outs, summed):
        assert_rel(o, s, FP32_REL, "summed")
    K.clip_accumulate(dgs, gclip, outs, accumulate=True)
    for o, s in zip(outs, summed):
        assert_rel(o, 2 * s, FP32_REL, "summed twice")


def test_clip_accumulate_bf16_in_fp32_out(K):
    torch.manual_seed(3)
    gs = [torch.randn(33, 24, 40).bfloat16(), torch.randn(33, 7).bfloat16()]
    _, clip, summed = O.clip_and_accumulate([g.float() for g in gs], 1.0)
    dgs = [dev(g) for g in gs]
    ss = K.sumsq_rows(dgs)
    _, gclip = K.clip_factor(ss, 1.0)
    assert_rel(gclip, clip, 1e-5)
    outs = [torch.empty(g.shape[1:], device="cuda") for g in gs]
    K.clip_accumulate(dgs, gclip, outs, accumulate=False)
    for o, s in zip(outs, summed):
        assert_rel(o, s, FP32_REL)
    outs16 = [torch.empty(g.shape[1:], device="cuda", dtype=torch.bfloat16) for g in gs]
    K.clip_accumulate(dgs, gclip, outs16, accumulate=False)
    for o, s in zip(outs16, summed):
        assert_rel(o, s, BF16_REL)


def test_clip_factor_from_norms(K):
    ns = torch.tensor([[3.0, 0.0, 0.3], [4.0, 0.0, 0.4]])
    norm, clip = K.clip_factor(dev(ns), 1.0, is_norm=True)
    assert_rel(norm, O.per_sample_norm(list(ns)), 1e-6)
    assert_rel(clip, O.clipping_coef(list(ns), 1.0), 1e-6)


def test_clip_accumulate_many_tensors(K):
    torch.manual_seed(4)
    gs = [torch.randn(6, 3 + i) for i in range(60)]  # more than one launch's worth
    _, clip, summed = O.clip_and_accumulate(gs, 2.0)
    dgs = [dev(g) for g in gs]
    _, gclip = K.clip_factor(K.sumsq_rows(dgs), 2.0)
    outs = [torch.empty(g.shape[1:], device="cuda") for g in gs]
    K.clip_accumulate(dgs, gclip, outs, accumulate=False)
    for o, s in zip(outs, summed):
        assert_rel(o, s, FP32_REL)


def test_clip_accumulate_very_large_tensors(K):
    """The shape for tensors past 8.4 M elements in total: blocks own 32768-element spans, so cover
    a ragged last span, a tensor shorter than one span, per-layer factors, fp32 and bf16
    gradients, and accumulation into a previous sum."""
    torch.manual_seed(41)
    n = 3
    sizes = [257 * 32768 + 4 * 1237, 1000, 2 * 32768]
    gs = [torch.randn(n, p) for p in sizes]
    dgs = [dev(g) for g in gs]
    clip = torch.tensor([[0.5, 1.0, 0.25], [1.0, 0.125, 0.75], [0.3, 0.6, 0.9]])
    want = [(c[:, None].double() * g.double()).sum(0) for c, g in zip(clip, gs)]
    outs = [torch.full((p,), float("nan"), device="cuda") for p in sizes]
    K.clip_accumulate(dgs, dev(clip), outs, accumulate=False)
    for o, w in zip(outs, want):
        assert_rel(o, w, FP32_REL, "very large, fresh")
    K.clip_accumulate(dgs, dev(clip), outs, accumulate=True)
    for o, w in zip(outs, want):
        assert_rel(o, 2 * w, FP32_REL, "very large, accumulated")
    shared = dev(clip[0].contiguous())
    K.clip_accumulate(dgs, shared, outs, accumulate=False)
    for o, g in zip(outs, gs):
        assert_rel(o, (clip[0][:, None].double() * g.double()).sum(0), FP32_REL, "very large, one factor row")
    g16 = [g.bfloat16() for g in gs]
    K.clip_accumulate([dev(g) for g in g16], shared, outs, accumulate=False)
    for o, g in zip(outs, g16):
        assert_rel(o, (clip[0][:, None].double() * g.double()).sum(0), FP32_REL, "very large, bf16 gradients")


def test_per_layer_clip_factors_and_accumulate(K):
    """[K, n] factor table: row k from parameter k's own norm and bound; bf16 and fp32 tensors,
    fresh and accumulating, more tensors than one launch holds."""
    torch.manual_seed(31)
    n = 9
    gs = [torch.randn(n, 5, 7), torch.randn(n, 33) * 3, torch.randn(n, 4, 2, 2) * 0.01]
    bounds = [0.5, 2.0, 1.0]
    want_clip, want = O.per_layer_clip_and_accumulate([g.double() for g in gs], bounds)
    dgs = [dev(g) for g in gs]
    clip = K.clip_factor_per_layer(K.sumsq_rows(dgs), bounds)
    assert clip.shape == (3, n)
    assert_rel(clip, torch.stack(want_clip), FP32_REL, "per-layer factors")
    outs = [torch.empty(g.shape[1:], device="cuda") for g in gs]
    K.clip_accumulate(dgs, clip, outs, accumulate=False)
    K.clip_accumulate(dgs, clip, outs, accumulate=True)
    for o, w in zip(outs, want):
        assert_rel(o, 2 * w, FP32_REL, "per-layer clipped sum, accumulated once")
    norms_in = K.clip_factor_per_layer(K.sumsq_rows(dgs).sqrt(), bounds, is_norm=True)
    assert torch.equal(norms_in, clip) or (norms_in - clip).abs().max() < 1e-6
    many = [torch.randn(4, 6) * (k + 1) for k in range(50)]
    mb = [0.1 * (k + 1) for k in range(50)]
    _, mwant = O.per_layer_clip_and_accumulate([g.double() for g in many], mb)
    dm = [dev(g) for g in many]
    mclip = K.clip_factor_per_layer(K.sumsq_rows(dm), mb)
    mouts = [torch.empty(6, device="cuda") for _ in many]
    K.clip_accumulate(dm, mclip, mouts, accumulate=False)
    for o, w in zip(mouts, mwant):
        assert_rel(o, w, FP32_REL)


def test_empty_batch_through_every_wrapper(K):
    """n == 0 (a Poisson draw can be empty): every wrapper returns tensors of the right shape with a
    leading zero and launches nothing that could fault."""
    e = lambda *shape, dtype=torch.float32: torch.empty(*shape, device="cuda", dtype=dtype)  # noqa: E731
    gs, ss = K.linear_grad_sample(e(0, 5), e(0, 7))
    assert gs.shape == (0, 5, 7) and ss.shape == (0,)
    assert K.linear_grad_sample(e(0, 3, 5), e(0, 3, 7))[0].shape == (0, 5, 7)
    assert K.linear_bias_grad_sample(e(0, 3, 5)).shape == (0, 5)
    nw, nb = K.linear_ghost_norm(e(0, 3, 5), e(0, 3, 7), want_bias=True)
    assert nw.shape == (0,) and nb.shape == (0,)
    assert K.conv2d_grad_sample(e(0, 2, 6, 6), e(0, 4, 4, 4), (3, 3), (1, 1), (0, 0, 0, 0), (1, 1), 1)[0].shape == (0, 4, 2, 3, 3)
    assert K.conv_bias_grad_sample(e(0, 4, 4, 4)).shape == (0, 4)
    ids = e(0, 6, dtype=torch.int64)
    assert K.embedding_grad_sample(ids, e(0, 6, 4), 9).shape == (0, 9, 4)
    assert K.embedding_ghost_norm(ids, e(0, 6, 4)).shape == (0,)
    assert K.embedding_bag_grad_sample(e(0, dtype=torch.int64), e(0, dtype=torch.int64), e(0, 4), 9).shape == (0, 9, 4)
    gw, gb = K.group_norm_grad_sample(e(0, 4, 5), e(0, 4, 5), 2, 1e-5)
    assert gw.shape == (0, 4) and gb.shape == (0, 4)
    assert K.rms_norm_grad_sample(e(0, 3, 8), e(0, 3, 8), 8, 1e-5).shape == (0, 8)
    assert K.layer_norm_grad_sample(e(0, 3, 8), e(0, 3, 8), 8, 1e-5)[0].shape == (0, 8)
    assert K.sumsq_rows([e(0, 5, 7), e(0, 3)]).shape == (2, 0)
    norm, clip = K.clip_factor(e(2, 0), 1.0)
    assert norm.shape == (0,) and clip.shape == (0,)
    assert K.clip_factor_per_layer(e(2, 0), [1.0, 2.0]).shape == (2, 0)
    fresh, kept = torch.full((5, 7), 3.0, device="cuda"), torch.full((3,), 3.0, device="cuda")
    K.clip_accumulate([e(0, 5, 7)], clip, [fresh], accumulate=False)
    K.clip_accumulate([e(0, 3)], clip, [kept], accumulate=True)
    assert fresh.abs().sum() == 0 and (kept == 3.0).all()  # an empty sum is zero; accumulating it changes nothing


# ---- Noise ---------------------------------------------------------------------------
def test_add_noise_zero_std_is_exact(K):
    torch.manual_seed(5)
    s = torch.randn(1003)
    out = torch.empty(1003, device="cuda")
    K.add_noise(dev(s), out, std=0.0, denom=1.0, seed=1, offset=0)
    assert torch.equal(out.cpu(), s)
    K.add_noise(dev(s), out, std=0.0, denom=256.0, seed=1, offset=0)
    assert torch.equal(out.cpu(), s / 256.0)


def test_noise_stream_matches_philox_restatement(K):
    P = 4099
    out = torch.empty(P, device="cuda")
    K.fill_normal(out, std=1.0, seed=0xDEADBEEFCAFE, offset=12345678901)
    want = O.philox_normal(P, seed=0xDEADBEEFCAFE, offset=12345678901)
    np.testing.assert_allclose(out.cpu().numpy(), want, rtol=0, atol=2e-5)


def test_noise_statistics(K):
    P = 1 << 22
    out = torch.empty(P, device="cuda")
    K.fill_normal(out, std=1.7, seed=42, offset=0)
    z = out.double()
    se = 1.7 / math.sqrt(P)
    assert abs(z.mean().item()) < 5 * se
    assert abs(z.std().item() - 1.7) < 5 * 1.7 / math.sqrt(2 * P)
    assert abs(((z / 1.7) ** 4).mean().item() - 3.0) < 0.03
    out2 = torch.empty(P, device="cuda")
    K.fill_normal(out2, std=1.7, seed=42, offset=1)
    assert abs(torch.corrcoef(torch.stack([out, out2]))[0, 1].item()) < 5 / math.sqrt(P)
    K.fill_normal(out2, std=1.7, seed=42, offset=0)
    assert torch.equal(out, out2)  # same (seed, offset) -> same bits


def test_add_noise_secure_draws_and_dtypes(K):
    P = 1 << 20
    s = torch.zeros(P, device="cuda")
    g = torch.empty(P, device="cuda")
    K.add_noise(s, g, std=2.0, denom=4.0, seed=3, offset=10, draws=4)
    assert abs(g.double().std().item() - 0.5) < 5e-3 and abs(g.double().mean().item()) < 5e-3
    gb = torch.empty(P, device="cuda", dtype=torch.bfloat16)
    K.add_noise(s.bfloat16(), gb, std=1.0, denom=1.0, seed=3, offset=10)
    assert abs(gb.double().std().item() - 1.0) < 1e-2


def test_add_noise_multi_is_one_stream_laid_across_the_tensors(K):
    """Tensor k's element i draws group (groups before k) + i // 4 of the restated stream; odd
    sizes (scalar tails), a 1-element tensor and a misaligned view are in the mix."""
    torch.manual_seed(11)
    sizes = [1030, 1, 7, 4096, 513]
    base = torch.randn(sum(sizes) + 64, device="cuda")
    summed, lo = [], 0
    for k, P in enumerate(sizes):
        start = lo + (1 if k == 2 else 0)  # tensor 2 starts 4 bytes off a 16-byte boundary
        summed.append(base[start : start + P])
        lo += P + 8 - (P % 4)
    grads = [torch.empty(P, device="cuda") for P in sizes]
    used = K.add_noise_multi(summed, grads, std=1.5, denom=8.0, seed=77, offset=40, draws=1)
    assert used == 1
    total_groups = sum((P + 3) // 4 for P in sizes)
    z = O.philox_normal(4 * total_groups, seed=77, offset=40)
    g0 = 0
    for P, s, g in zip(sizes, summed, grads):
        want = (s.cpu().numpy() + np.float32(1.5) * z[4 * g0 : 4 * g0 + P]) / np.float32(8.0)
        np.testing.assert_allclose(g.cpu().numpy(), want, rtol=0, atol=1e-5)
        g0 += (P + 3) // 4
    # more tensors than one launch holds: later launches move on by `draws` offsets
    many = [torch.zeros(5, device="cuda") for _ in range(50)]
    outs = [torch.empty(5, device="cuda") for _ in range(50)]
    assert K.add_noise_multi(many, outs, std=1.0, denom=1.0, seed=1, offset=8, draws=1) == 2
    z8, z9 = O.philox_normal(8 * 48, seed=1, offset=8), O.philox_normal(16, seed=1, offset=9)
    np.testing.assert_allclose(outs[47].cpu().numpy(), z8[8 * 47 : 8 * 47 + 5], rtol=0, atol=2e-5)
    np.testing.assert_allclose(outs[49].cpu().numpy(), z9[8:13], rtol=0, atol=2e-5)
    # std == 0 is exact
    K.add_noise_multi(summed, grads, std=0.0, denom=1.0, seed=0, offset=0)
    for s, g in zip(summed, grads):
        assert torch.equal(s, g)


# ---- Linear ghost norms --------------------------------------------------------------
GHOST_SHAPES = [
    # (n, T, in, out)
    (5, 1, 40, 24),  # closed form
    (3, 2, 8, 4),
    (4, 9, 33, 17),  # odd everything -> scalar loads
    (2, 64, 128, 64),  # exactly one 64-tile
    (3, 100, 72, 200),  # 128-tiles, ragged T, one tile pair
    (2, 300, 136, 264),  # 3 x 3 tile pairs, off-diagonal weights
    (1, 512, 1024, 256),
]


# "gram": sum over the T x T Grams (the reference's formula); "direct": the squared norm of the
# per-sample gradient tiles as they are formed; "auto": the library's choice by cost
GHOST_ROUTES = [0, 1, 2]  # DPK_ROUTE_AUTO, DPK_ROUTE_GRAM, DPK_ROUTE_DIRECT


@pytest.mark.parametrize(
    "n,T,fin,fout",
    GHOST_SHAPES
    + [(3, 200, 256, 16), (2, 130, 8, 520)]  # thin layers: the direct route by choice
    # feature sizes that are multiples of 32: the direct-load kernel on fp32 operands (route "gram")
    + [(3, 200, 64, 96), (2, 300, 160, 288), (5, 1000, 32, 64)]
    # ... with a tail cut into pieces along k: few units (all in pieces), 576 units (512 whole tiles + 64 units in 4 pieces each)
    + [(2, 256, 512, 256), (3, 150, 64, 64), (16, 1000, 64, 128)],
)
@pytest.mark.parametrize("scale", [1.0, 4.0])
@pytest.mark.parametrize("route", GHOST_ROUTES)
def test_linear_ghost_norm_f32(K, n, T, fin, fout, scale, route):
    torch.manual_seed(T * 7 + fin)
    a = torch.randn(n, T, fin)
    b = torch.randn(n, T, fout) * 0.1
    # float64 oracle on the 3-d Gram path, and its identity with the materialised gradient
    want_w, want_b = O.linear_norm_sample(a.double(), (b * scale).double())
    gs_w, gs_b = O.linear_grad_sample(a.double(), (b * scale).double())
    torch.testing.assert_close(want_w, gs_w.flatten(1).norm(dim=1), rtol=1e-9, atol=1e-12)
    nw, nb = K.linear_ghost_norm(dev(b), dev(a), scale=scale, want_weight=True, want_bias=True, route=route)
    assert nw.dtype == torch.float32
    assert_rel(nw, want_w, FP32_REL, "weight norm")
    assert_rel(nb, want_b, FP32_REL, "bias norm")
    only_b = K.linear_ghost_norm(dev(b), dev(a), scale=scale, want_weight=False, want_bias=True, route=route)
    assert only_b[0] is None
    assert_rel(only_b[1], want_b, FP32_REL, "bias norm alone")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize(
    "n,layers",
    [
        # (T, in, out, want_w, want_b): pooled tile layers of two lengths, a thin layer (direct route),
        # odd feature sizes (register-staged kernel), T = 1, a bias-only layer
        (3, [(200, 64, 128, True, True), (200, 128, 64, True, False), (130, 1024, 16, True, True),
             (70, 40, 24, True, True), (1, 96, 64, True, True), (300, 64, 192, False, True)]),
        # 16 samples: two per XCD; units of three layer shapes in one launch, ragged T
        (16, [(1000, 64, 128, True, True), (1000, 128, 64, True, True), (520, 192, 64, True, False)]),
        # 5 samples: XCDs with one sample and XCDs with none
        (5, [(256, 128, 128, True, True), (256, 64, 256, True, True)]),
        # 32 samples, 10 + 10 tile pairs each: 80 units per XCD = one round of 64 and a tail of 16 cut into pieces along k
        (32, [(512, 64, 128, True, True), (512, 128, 64, True, True)]),
    ],
)
def test_linear_ghost_norm_multi_matches_layer_by_layer(K, dtype, n, layers):
    """All layers of a pass in one call (the tile pairs of every layer share the launch, longest
    first, the tail as pieces along k) against the float64 oracle and against one call per layer."""
    torch.manual_seed(n * 31 + len(layers))
    items, wants, singles = [], [], []
    for T, fin, fout, want_w, want_b in layers:
        a = torch.randn(n, T, fin).to(dtype)
        b = (torch.randn(n, T, fout) * 0.1).to(dtype)
        scale = 2.0 if fin == 64 else 1.0
        ow, ob = O.linear_norm_sample(a.double(), (b.double() * scale))
        nw = torch.full((n,), float("nan"), device="cuda") if want_w else None
        nb = torch.full((n,), float("nan"), device="cuda") if want_b else None
        items.append((dev(b), dev(a), scale, nw, nb))
        wants.append((ow if want_w else None, ob if want_b else None))
        singles.append(K.linear_ghost_norm(dev(b), dev(a), scale=scale, want_weight=want_w, want_bias=want_b))
    K.linear_ghost_norm_multi(items)
    bar = FP32_REL if dtype == torch.float32 else 1e-4  # bf16 inputs are exact, accumulation is fp32
    for (_, _, _, nw, nb), (ow, ob), (sw, sb), lay in zip(items, wants, singles, layers):
        for got, want, single, what in ((nw, ow, sw, "weight"), (nb, ob, sb, "bias")):
            if want is None:
                assert got is None
                continue
            assert_rel(got, want, bar, f"{what} norm of layer {lay}")
            assert_rel(got, single, FP32_REL, f"{what} norm of layer {lay} against its own launch")


@pytest.mark.parametrize("count", [40, 300])
def test_linear_ghost_norm_multi_many_layers(K, count):
    """More layers than one pooled launch takes (32) and more than one call's table (256)."""
    torch.manual_seed(count)
    n, T = 2, 128
    items, wants = [], []
    for k in range(count):
        fin, fout = (64, 128) if k % 3 else (128, 64)
        a = torch.randn(n, T, fin).bfloat16()
        b = (torch.randn(n, T, fout) * 0.1).bfloat16()
        ow, ob = O.linear_norm_sample(a.double(), b.double())
        nw = torch.full((n,), float("nan"), device="cuda")
        nb = torch.full((n,), float("nan"), device="cuda") if k % 2 else None
        items.append((dev(b), dev(a), 1.0, nw, nb))
        wants.append((ow, ob if k % 2 else None))
    K.linear_ghost_norm_multi(items)
    for k, ((_, _, _, nw, nb), (ow, ob)) in enumerate(zip(items, wants)):
        assert_rel(nw, ow, 1e-4, f"weight norm of layer {k}")
        if ob is not None:
            assert_rel(nb, ob, 1e-4, f"bias norm of layer {k}")


def test_float16_tensors_go_through_the_float32_kernels(K):
    """float16 has no kernels of its own: the optimizer wrappers widen (exactly) and narrow the
    result, so they agree to the bit with the float32 call on the widened tensors, rounded once."""
    torch.manual_seed(9)
    n, P = 5, 300
    gs = dev(torch.randn(n, P).half())
    clip = dev(torch.rand(n))
    assert torch.equal(K.sumsq_rows([gs]), K.sumsq_rows([gs.float()]))
    out16, out32 = torch.empty(P, device="cuda", dtype=torch.float16), torch.empty(P, device="cuda")
    K.clip_accumulate([gs], clip, [out16], False)
    K.clip_accumulate([gs.float()], clip, [out32], False)
    assert torch.equal(out16, out32.half())
    base = out32.half().float()
    K.clip_accumulate([gs], clip, [out16], True)  # accumulates onto the float16 value
    K.clip_accumulate([gs.float()], clip, [base], True)
    assert torch.equal(out16, base.half())
    g16, g32 = torch.empty_like(out16), torch.empty_like(out32)
    K.add_noise(out16, g16, 0.5, 4.0, 123, 8)
    K.add_noise(out16.float(), g32, 0.5, 4.0, 123, 8)
    assert torch.equal(g16, g32.half())
    assert K.add_noise_multi([out16], [g16], 0.5, 4.0, 123, 8) == 1 and torch.equal(g16, g32.half())
    assert K.supported_dtype(torch.float16) and not K.native_dtype(torch.float16)
    with pytest.raises(TypeError):
        K.linear_grad_sample(dev(torch.randn(2, 4).half()), dev(torch.randn(2, 4).half()))


WEIGHTED_SUM_CASES = [
    # (n, T, in, out, pieces)
    (8, 32, 128, 128, 1),  # one k tile per sample: a rescaling before every tile
    (8, 64, 512, 256, 4),
    (16, 128, 256, 512, None),  # the wrapper's own choice of pieces
    (6, 96, 72, 136, 2),  # ragged block tiles, three k tiles per sample
    (4, 256, 1024, 1024, 1),
    (3, 32, 2048, 2048, 1),  # enough output tiles for the 256-wide block tile
]


@pytest.mark.parametrize("n,T,fin,fout,pieces", WEIGHTED_SUM_CASES)
@pytest.mark.parametrize("coefs", ["spread", "equal", "tiny_and_zero", "zeros_after_large_sums"])
@pytest.mark.parametrize("out_f32", [False, True])
def test_linear_weighted_sum(K, n, T, fin, fout, pieces, coefs, out_f32):
    """sum_n coef[n] * b[n]^T a[n] with the coefficients applied to the accumulators, against the
    oracle's per-sample gradients weighted and added in fp64."""
    torch.manual_seed(n * 100 + T + fin)
    a = torch.randn(n, T, fin).bfloat16()
    b = (torch.randn(n, T, fout) * 0.1).bfloat16()
    if coefs == "spread":
        c = torch.rand(n) * 0.99 + 0.01
    elif coefs == "equal":
        c = torch.full((n,), 0.37)
    elif coefs == "zeros_after_large_sums":
        # masked samples (coefficient exactly 0) after partial sums of 1e10 and more: a sample that
        # counts zero times must leave the sum alone (dividing the accumulator by a floored
        # coefficient would overflow here); zeros first, last and in a row as well
        a, b = (a.float() * 3e4).bfloat16(), (b.float() * 3e5).bfloat16()
        c = torch.rand(n) * 0.5 + 0.5
        c[1], c[-1] = 0.0, 0.0
        if n > 4:
            c[0], c[3], c[4] = 0.0, 0.0, 1e-38
    else:  # coefficients twelve orders of magnitude apart and an exact zero, at either end too
        c = torch.rand(n) * 0.9 + 0.1
        c[0], c[n // 2], c[-1] = 1e-12, 0.0, 3e-9
    gs, _ = O.linear_grad_sample(a.double(), b.double())
    want = (c.double().view(n, 1, 1) * gs.double()).sum(0) * 2.0
    got = K.linear_weighted_sum(
        dev(b), dev(a), dev(c), scale=2.0, pieces=pieces, out_dtype=torch.float32 if out_f32 else None
    )
    assert got.shape == (fout, fin) and got.dtype == (torch.float32 if out_f32 else torch.bfloat16)
    # bf16 inputs are exact and accumulation is fp32; a bf16 result is rounded once
    assert_rel(got[None], want[None], 1e-4 if out_f32 else BF16_REL, "weighted sum")


@pytest.mark.parametrize("count", [3, 40])
def test_linear_weighted_sum_multi(K, count):
    """Several layers pooled into one launch (more than one launch's table for 40), with
    different shapes, batch sizes and sequence lengths: each sum as the single-layer call
    gives it (one piece), and against the oracle for the first."""
    torch.manual_seed(count)
    shapes = [(8, 64, 128, 256), (4, 32, 512, 136), (6, 96, 72, 264), (16, 32, 256, 2048)]
    items = []
    for k in range(count):
        n, T, fin, fout = shapes[k % len(shapes)]
        a = dev(torch.randn(n, T, fin).bfloat16())
        b = dev((torch.randn(n, T, fout) * 0.1).bfloat16())
        c = dev(torch.rand(n) * 0.9 + 0.1)
        items.append((b, a, c, 1.0 + k % 3))
    for out_dtype in (None, torch.float32):
        sums = K.linear_weighted_sum_multi(items, out_dtype=out_dtype, pooled=True)
        assert len(sums) == count
        for (b, a, c, scale), got in zip(items, sums):
            want = K.linear_weighted_sum(b, a, c, scale=scale, pieces=1, out_dtype=out_dtype)
            assert got.dtype == want.dtype and got.shape == want.shape
            # the pool may choose the other block tile: same products, another order of addition
            assert_rel(got[None], want[None], 1e-5 if out_dtype else BF16_REL, "pooled against single")
    b, a, c, scale = items[0]
    gs, _ = O.linear_grad_sample(a.cpu().double(), b.cpu().double())
    want = (c.cpu().double().view(-1, 1, 1) * gs).sum(0) * scale
    assert_rel(K.linear_weighted_sum_multi(items[:1], out_dtype=torch.float32, pooled=True)[0][None], want[None], 1e-4, "pooled against the oracle")
    assert K.linear_weighted_sum_multi([]) == []
    with pytest.raises(RuntimeError, match="dpk_linear_weighted_sum_multi"):
        K.linear_weighted_sum_multi([(b[:, :16].contiguous(), a[:, :16].contiguous(), c, 1.0)], pooled=True)


def test_linear_weighted_sum_keeps_a_nan_and_multi_refuses_other_shapes(K):
    torch.manual_seed(5)
    a, b = dev(torch.randn(4, 32, 128).bfloat16()), dev(torch.randn(4, 32, 128).bfloat16())
    c = torch.tensor([0.5, float("nan"), 0.25, 1.0])
    assert torch.isnan(K.linear_weighted_sum(b, a, dev(c))).all()
    assert not K.linear_weighted_sum_takes(b[:, :16], a[:, :16])  # half a k tile per sample
    assert not K.linear_weighted_sum_takes(b.float(), a.float())
    assert not K.linear_weighted_sum_takes(b[..., :64], a)
    with pytest.raises(RuntimeError, match="dpk_linear_weighted_sum_multi"):  # the pool takes the bf16 kernel's shapes only
        K.linear_weighted_sum_multi([(b[:, :16].contiguous(), a[:, :16].contiguous(), dev(c), 1.0)])
    with pytest.raises(RuntimeError, match="dpk_linear_weighted_sum"):
        K.linear_weighted_sum(b, a, dev(c), pieces=0)
    with pytest.raises(TypeError):
        K.linear_weighted_sum(b.half(), a.half(), dev(c))


# fp32 operands, positions that are not whole k tiles, odd feature sizes, misaligned tensors: the fp32
# MFMA kernel with weighted rows
GENERIC_WSUM_CASES = [
    # (n, mid, in, out, dtype, pieces)
    (5, (7,), 24, 40, torch.float32, 1),
    (6, (33,), 136, 200, torch.float32, None),
    (3, (4, 5), 30, 18, torch.float32, 1),  # odd sizes: element-wise loads
    (8, (64,), 256, 128, torch.float32, 4),
    (4, (50,), 128, 256, torch.bfloat16, None),  # bf16, 50 positions per sample
    (2, (31,), 72, 100, torch.bfloat16, 2),
    (7, (1,), 64, 32, torch.float32, 1),  # one position per sample
    (3, (), 48, 16, torch.float32, 1),  # 2-d input
    # fp32 with whole k tiles of 16 positions: the direct-load fp32 kernel, coefficients on its accumulators
    (8, (16,), 128, 128, torch.float32, 1),  # one k tile per sample: a rescaling before every tile
    (6, (48,), 136, 200, torch.float32, 2),  # ragged block tiles
    (16, (128,), 512, 256, torch.float32, None),
    (4, (80,), 1024, 1024, torch.float32, 1),
]


@pytest.mark.parametrize("n,mid,fin,fout,dtype,pieces", GENERIC_WSUM_CASES)
@pytest.mark.parametrize("coefs", ["spread", "tiny_and_zero"])
def test_linear_weighted_sum_generic_shapes(K, n, mid, fin, fout, dtype, pieces, coefs):
    """sum_n coef[n] * b[n]^T a[n] and the bias sum for everything the bf16 tile kernel does not
    take, against (coef * gs).sum(0) of the oracle's per-sample gradients in fp64: fp32 1e-5, bf16
    inputs exact products with fp32 accumulation (1e-5 into an fp32 result, one rounding into bf16)."""
    torch.manual_seed(n * 31 + fin)
    a = torch.randn(n, *mid, fin).to(dtype)
    b = (torch.randn(n, *mid, fout) * 0.3).to(dtype)
    c = torch.rand(n) * 0.99 + 0.01
    if coefs == "tiny_and_zero":
        c[0], c[n // 2], c[-1] = 1e-12, 0.0, 3e-9
    assert not K.linear_weighted_sum_takes(dev(b), dev(a))
    gs_w, gs_b = O.linear_grad_sample(a.double(), b.double())
    want_w = (c.double().view(n, 1, 1) * gs_w).sum(0) * 1.5
    want_b = (c.double().view(n, 1) * gs_b).sum(0) * 1.5
    for out_dtype in (None, torch.float32):
        got = K.linear_weighted_sum(dev(b), dev(a), dev(c), scale=1.5, pieces=pieces, out_dtype=out_dtype)
        assert got.shape == (fout, fin) and got.dtype == (out_dtype or dtype)
        bar = BF16_REL if (out_dtype or dtype) == torch.bfloat16 else FP32_REL
        assert_rel(got[None], want_w[None], bar, f"weighted sum {dtype} -> {got.dtype}")
        got_b = K.linear_bias_weighted_sum(dev(b), dev(c), scale=1.5, out_dtype=out_dtype)
        assert got_b.shape == (fout,) and got_b.dtype == (out_dtype or dtype)
        assert_rel(got_b, want_b, bar, f"bias weighted sum {dtype} -> {got_b.dtype}")
    if dtype == torch.bfloat16:
        # operands two bytes off a 16-byte boundary take the same path
        odd_b = torch.empty(b.numel() + 1, dtype=dtype, device="cuda")[1:].view(b.shape).copy_(b)
        got = K.linear_weighted_sum(odd_b, dev(a), dev(c), scale=1.5, pieces=pieces, out_dtype=torch.float32)
        assert_rel(got[None], want_w[None], FP32_REL, "misaligned backprops")


def test_linear_bias_weighted_sum_at_benchmark_width(K):
    """C3's first layer: 32 x 512 rows of 4096 bf16 columns, 64 chunks of rows."""
    torch.manual_seed(2)
    n, T, D = 32, 512, 4096
    b = (torch.randn(n, T, D) * 0.02).bfloat16()
    c = torch.rand(n) * 0.9 + 0.1
    want = (c.double().view(n, 1, 1) * b.double()).sum((0, 1))
    assert_rel(K.linear_bias_weighted_sum(dev(b), dev(c), out_dtype=torch.float32), want, 1e-5, "bias weighted sum")
    assert_rel(K.linear_bias_weighted_sum(dev(b), dev(c)), want, BF16_REL, "bias weighted sum bf16")


@pytest.mark.parametrize(
    "n,Tshape,V,D,dtype",
    [(5, (3, 2), 9, 4, torch.float32), (3, (40,), 7, 17, torch.float32), (4, (300,), 50, 64, torch.bfloat16),
     (2, (64,), 10, 1030, torch.float32), (6, (1000,), 3000, 128, torch.bfloat16), (3, (2000,), 11, 8, torch.float32),
     (1, (1,), 1, 4, torch.float32), (40, (1000,), 50000, 8, torch.float32), (9, (4097,), 300, 4, torch.float32),
     (5, (1023,), 2, 4, torch.float32)],
)
def test_embedding_weighted_sum(K, n, Tshape, V, D, dtype):
    """out[v] = sum_n coef[n] sum_{t: ids[n,t]==v} b[n,t]: the clip-weighted sum of the Embedding
    per-sample gradients, against the oracle's [n, V, D] gradients weighted and added in fp64
    (ids repeated inside a sample and across samples; the batch of up to 40000 positions is sorted in
    runs of 1024 or 4096 that are merged by binary search). Which rows are written is index work:
    exact. Two runs give the same bits."""
    torch.manual_seed(V * 7 + D)
    ids = torch.randint(0, V, (n, *Tshape))
    b = torch.randn(n, *Tshape, D).to(dtype)
    c = torch.rand(n) * 0.9 + 0.1
    if n > 2:
        c[1] = 0.0
    gs = O.embedding_grad_sample(ids, b.double(), V)
    want = (c.double().view(n, 1, 1) * gs).sum(0) * 0.5
    K.check_embedding_indices("cuda")
    for out_dtype in (None, torch.float32):
        got = K.embedding_weighted_sum(dev(ids), dev(b), dev(c), V, scale=0.5, out_dtype=out_dtype)
        assert got.shape == (V, D) and got.dtype == (out_dtype or dtype)
        # rows as the groups of the comparison: every table row is held to its own size
        assert_rel(got, want, BF16_REL if got.dtype == torch.bfloat16 else FP32_REL, f"embedding weighted sum -> {got.dtype}")
        named = torch.zeros(V, dtype=torch.bool)
        named[ids.reshape(-1)] = True
        assert not got.cpu()[~named].any(), "a row no id names was written"
        again = K.embedding_weighted_sum(dev(ids), dev(b), dev(c), V, scale=0.5, out_dtype=out_dtype)
        assert torch.equal(got, again)
    K.check_embedding_indices("cuda")
    # an id outside the table contributes nothing and raises the flag
    bad = ids.clone()
    bad.view(-1)[0] = V
    got = K.embedding_weighted_sum(dev(bad), dev(b), dev(c), V, out_dtype=torch.float32)
    with pytest.raises(IndexError, match="outside"):
        K.check_embedding_indices("cuda")
    keep = torch.ones(ids.numel(), dtype=torch.bool)
    keep[0] = False
    want2 = torch.zeros(V, D, dtype=torch.float64)
    want2.index_add_(0, ids.reshape(-1)[keep], (c.double().repeat_interleave(ids[0].numel()).view(-1, 1) * b.double().reshape(-1, D))[keep])
    assert_rel(got, want2, FP32_REL if dtype == torch.float32 else 1e-4, "with one id out of range")


def test_linear_ghost_norm_2d_inputs(K):
    torch.manual_seed(21)
    a, b = torch.randn(6, 50), torch.randn(6, 30)
    want_w, want_b = O.linear_norm_sample(a, b)
    nw, nb = K.linear_ghost_norm(dev(b), dev(a), want_bias=True)
    assert_rel(nw, want_w, FP32_REL)
    assert_rel(nb, want_b, FP32_REL)


@pytest.mark.parametrize(
    "n,T,fin,fout",
    [
        (3, 2, 8, 16),
        (2, 70, 40, 24),
        (2, 200, 136, 264),
        (2, 256, 1024, 512),  # direct-to-LDS kernel, few units: every unit cut into pieces along k
        (3, 33, 30, 18),
        (3, 150, 64, 64),  # tail pieces of tiles that reach beyond T
        (3, 200, 64, 128),  # tail pieces with a few valid rows
        (20, 640, 64, 64),  # 300 units on a 256-CU device: whole-tile blocks only
        (16, 1000, 64, 128),  # 576 units: 512 whole-tile blocks and a tail in pieces, ragged T
        (4, 512, 1024, 16),  # a low-rank adapter: thin on one side
        (4, 512, 16, 1024),
    ],
)
@pytest.mark.parametrize("route", GHOST_ROUTES)
def test_linear_ghost_norm_bf16(K, n, T, fin, fout, route):
    torch.manual_seed(T)
    a = torch.randn(n, T, fin).bfloat16()
    b = (torch.randn(n, T, fout) * 0.02).bfloat16()
    want_w, want_b = O.linear_norm_sample(a.double(), b.double())
    nw, nb = K.linear_ghost_norm(dev(b), dev(a), want_weight=True, want_bias=True, route=route)
    # inputs are exact in bf16 and accumulation is fp32: far inside the bf16 bar
    assert_rel(nw, want_w, 1e-4, "weight norm bf16")
    assert_rel(nb, want_b, 1e-4, "bias norm bf16")


# ---- Conv2d ---------------------------------------------------------------------------
CONV_CASES = [
    dict(n=3, C=3, O=4, k=(3, 3), stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=1, H=6, W=7),
    dict(n=3, C=4, O=6, k=(3, 2), stride=(2, 1), padding=(0, 2), dilation=(1, 2), groups=2, H=9, W=8),
    dict(n=2, C=2, O=2, k=(2, 3), stride=(1, 2), padding="same", dilation=(2, 1), groups=1, H=7, W=9),
    dict(n=2, C=6, O=3, k=(1, 1), stride=(1, 1), padding="valid", dilation=(1, 1), groups=3, H=4, W=4),
    dict(n=4, C=1, O=16, k=(8, 8), stride=(2, 2), padding=(3, 3), dilation=(1, 1), groups=1, H=28, W=28),  # C1 conv1
    dict(n=4, C=16, O=32, k=(4, 4), stride=(2, 2), padding=(0, 0), dilation=(1, 1), groups=1, H=13, W=13),  # C1 conv2
    dict(n=2, C=64, O=64, k=(3, 3), stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=1, H=32, W=32),  # C4
    dict(n=2, C=24, O=160, k=(3, 3), stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=1, H=10, W=12),  # 128-tiles
    dict(n=2, C=16, O=16, k=(3, 3), stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=16, H=8, W=8),  # depthwise
    dict(n=2, C=16, O=24, k=(3, 3), stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=1, H=56, W=56),  # a patch above 64 KB of LDS
    dict(n=2, C=16, O=24, k=(3, 3), stride=(2, 2), padding=(1, 1), dilation=(1, 1), groups=1, H=56, W=52),
]


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("scale", [1.0, 2.0])
def test_conv2d_grad_sample_f32(K, case, scale):
    torch.manual_seed(case["C"] * 31 + case["O"])
    n = case["n"]
    x = torch.randn(n, case["C"], case["H"], case["W"])
    pad = O.conv2d_padding(case["padding"], case["k"], case["dilation"])
    oh = (case["H"] + pad[0] + pad[1] - (case["dilation"][0] * (case["k"][0] - 1) + 1)) // case["stride"][0] + 1
    ow = (case["W"] + pad[2] + pad[3] - (case["dilation"][1] * (case["k"][1] - 1) + 1)) // case["stride"][1] + 1
    b = torch.randn(n, case["O"], oh, ow)
    want_w, want_b = O.conv2d_grad_sample(
        x.double(), (b * scale).double(), kernel_size=case["k"], padding=case["padding"], stride=case["stride"],
        dilation=case["dilation"], groups=case["groups"],
    )
    gs, sumsq = K.conv2d_grad_sample(dev(x), dev(b), case["k"], case["stride"], pad, case["dilation"], case["groups"], scale=scale)
    assert_rel(gs, want_w, FP32_REL, "conv weight")
    assert_rel(sumsq, want_w.flatten(1).pow(2).sum(1), 2e-5, "conv sumsq")
    assert_rel(K.conv_bias_grad_sample(dev(b), scale=scale), want_b, FP32_REL, "conv bias")


# bf16 input runs its own kernel (bf16 MFMA; the gathered operand read in groups of 8, 4, 2 or 1
# positions according to the output width and stride): every group size, row-wise and chunked
# staging of the patch, ragged last trips of the k loop, misaligned backprops
CONV_BF16_EXTRA = [
    dict(n=2, C=8, O=12, k=(3, 3), stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=1, H=9, W=9),     # groups of 1
    dict(n=2, C=8, O=70, k=(3, 3), stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=1, H=5, W=6),     # groups of 2, Q % 4 != 0
    dict(n=2, C=12, O=20, k=(3, 3), stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=1, H=7, W=12),   # groups of 4
    dict(n=2, C=12, O=20, k=(3, 3), stride=(1, 1), padding=(1, 1), dilation=(1, 1), groups=2, H=10, W=24),  # groups of 8
    dict(n=2, C=5, O=9, k=(3, 5), stride=(1, 1), padding=(0, 3), dilation=(2, 2), groups=1, H=12, W=18),    # dilated, groups of 8
    dict(n=2, C=4, O=8, k=(1, 3), stride=(1, 1), padding=(0, 1), dilation=(1, 1), groups=1, H=1, W=200),    # a Conv1d's shape
]


@pytest.mark.parametrize("case", CONV_CASES + CONV_BF16_EXTRA)
@pytest.mark.parametrize("out_f32", [False, True])
def test_conv2d_grad_sample_bf16(K, case, out_f32):
    torch.manual_seed(case["C"] * 31 + case["O"] + 5)
    n = case["n"]
    x = torch.randn(n, case["C"], case["H"], case["W"]).bfloat16()
    pad = O.conv2d_padding(case["padding"], case["k"], case["dilation"])
    oh = (case["H"] + pad[0] + pad[1] - (case["dilation"][0] * (case["k"][0] - 1) + 1)) // case["stride"][0] + 1
    ow = (case["W"] + pad[2] + pad[3] - (case["dilation"][1] * (case["k"][1] - 1) + 1)) // case["stride"][1] + 1
    b = torch.randn(n, case["O"], oh, ow).bfloat16()
    want_w, _ = O.conv2d_grad_sample(
        x.double(), (b.double() * 0.5), kernel_size=case["k"], padding=case["padding"], stride=case["stride"],
        dilation=case["dilation"], groups=case["groups"],
    )
    gs, sumsq = K.conv2d_grad_sample(
        dev(x), dev(b), case["k"], case["stride"], pad, case["dilation"], case["groups"], scale=0.5,
        out_dtype=torch.float32 if out_f32 else None,
    )
    assert gs.dtype == (torch.float32 if out_f32 else torch.bfloat16)
    # exact products of bf16 inputs, fp32 accumulation: only a bf16 output rounds
    assert_rel(gs, want_w, FP32_REL if out_f32 else BF16_REL, "conv weight bf16")
    assert_rel(sumsq, want_w.flatten(1).pow(2).sum(1), 2e-5, "conv sumsq bf16")
    # the same launch without storing the gradient
    none, sumsq_only = K.conv2d_grad_sample(dev(x), dev(b), case["k"], case["stride"], pad, case["dilation"], case["groups"],
                                            scale=0.5, norm_only=True)
    assert none is None
    assert_rel(sumsq_only, want_w.flatten(1).pow(2).sum(1), 2e-5, "conv sumsq bf16, norm only")
    # backprops that start 2 bytes off a 16-byte boundary take the element-wise loads
    odd = torch.empty(b.numel() + 1, dtype=torch.bfloat16, device="cuda")[1:].view(b.shape).copy_(b)
    gs2, _ = K.conv2d_grad_sample(dev(x), odd, case["k"], case["stride"], pad, case["dilation"], case["groups"], scale=0.5,
                                  out_dtype=torch.float32 if out_f32 else None)
    assert torch.equal(gs2, gs)


CONV3D_GPU_CASES = [
    dict(n=3, C=2, O=3, k=(2, 3, 2), stride=(1, 1, 1), padding=(0, 1, 0), dilation=(1, 1, 1), groups=1, size=(4, 5, 6)),
    dict(n=2, C=4, O=4, k=(3, 2, 2), stride=(2, 1, 2), padding=(1, 0, 2), dilation=(1, 2, 1), groups=2, size=(6, 5, 7)),
    dict(n=2, C=2, O=2, k=(2, 2, 3), stride=(1, 1, 1), padding="same", dilation=(2, 1, 1), groups=1, size=(5, 4, 6)),
    dict(n=2, C=8, O=80, k=(3, 3, 3), stride=(1, 1, 1), padding=(1, 1, 1), dilation=(1, 1, 1), groups=1, size=(6, 8, 8)),  # 128-tiles
]


@pytest.mark.parametrize("case", CONV3D_GPU_CASES)
def test_conv3d_grad_sample_f32(K, case):
    torch.manual_seed(case["C"] * 7 + case["O"])
    n = case["n"]
    x = torch.randn(n, case["C"], *case["size"])
    pads = []
    for d in range(3):
        if case["padding"] == "same":
            total = case["dilation"][d] * (case["k"][d] - 1)
            pads.append((total // 2, total - total // 2))
        else:
            pads.append((case["padding"][d], case["padding"][d]))
    out = [
        (case["size"][d] + pads[d][0] + pads[d][1] - (case["dilation"][d] * (case["k"][d] - 1) + 1)) // case["stride"][d] + 1
        for d in range(3)
    ]
    b = torch.randn(n, case["O"], *out)
    want_w, want_b = O.conv3d_grad_sample(
        x.double(), (b * 2.0).double(), kernel_size=case["k"], padding=case["padding"], stride=case["stride"],
        dilation=case["dilation"], groups=case["groups"],
    )
    gs, sumsq = K.conv3d_grad_sample(dev(x), dev(b), case["k"], case["stride"], tuple(pads), case["dilation"], case["groups"], scale=2.0)
    assert_rel(gs, want_w, FP32_REL, "conv3d weight")
    assert_rel(sumsq, want_w.flatten(1).pow(2).sum(1), 2e-5, "conv3d sumsq")
    assert_rel(K.conv_bias_grad_sample(dev(b), scale=2.0), want_b, FP32_REL, "conv3d bias")


@pytest.mark.parametrize(
    "n,C,H,W,O,k,stride,pad,groups",
    [
        # few kernel elements, many output positions: blocks < 2 x CUs, so the contraction over the
        # positions is cut into pieces whose raw tiles a second kernel adds (ragged last piece)
        (4, 3, 96, 96, 64, 7, 2, 3, 1),
        (3, 2, 70, 66, 24, 3, 1, 1, 1),
        (2, 4, 64, 64, 8, 3, 1, 1, 2),
        # the same machinery is not taken for a layer with enough blocks or a short contraction
        (8, 16, 12, 12, 16, 3, 1, 1, 1),
    ],
)
def test_conv2d_split_contraction_and_norm_only(K, n, C, H, W, O, k, stride, pad, groups):
    torch.manual_seed(C * 100 + H)
    x = torch.randn(n, C, H, W)
    oh, ow = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    b = torch.randn(n, O, oh, ow)
    want_w, _ = O_conv(x, b, k, stride, pad, groups)
    geo = dict(kernel_size=(k, k), stride=(stride, stride), padding=(pad, pad, pad, pad), dilation=(1, 1), groups=groups)
    gs, sumsq = K.conv2d_grad_sample(dev(x), dev(b), scale=2.0, **geo)
    assert_rel(gs, 2.0 * want_w, FP32_REL, "conv gs")
    want_ss = (2.0 * want_w).double().flatten(1).pow(2).sum(1)
    assert_rel(sumsq, want_ss, FP32_REL, "conv sumsq")
    none, ss_only = K.conv2d_grad_sample(dev(x), dev(b), scale=2.0, norm_only=True, **geo)
    assert none is None
    assert_rel(ss_only, want_ss, FP32_REL, "conv sumsq, norm only")
    # bf16 inputs through the same kernels
    gs16, ss16 = K.conv2d_grad_sample(dev(x.bfloat16()), dev(b.bfloat16()), **geo)
    want16, _ = O_conv(x.bfloat16().float(), b.bfloat16().float(), k, stride, pad, groups)
    assert_rel(gs16, want16, BF16_REL, "conv gs bf16")
    assert_rel(ss16, want16.double().flatten(1).pow(2).sum(1), 1e-4, "conv sumsq bf16 (fp32 accumulators)")


def O_conv(x, b, k, stride, pad, groups):
    return O.conv2d_grad_sample(
        x.double(), b.double(), kernel_size=(k, k), padding=(pad, pad), stride=(stride, stride), dilation=(1, 1), groups=groups
    )



# ---- Embedding ------------------------------------------------------------------------
def test_embedding_golden_vectors(K, embedding_norm_cases):
    """The reference's own known-answer triples and docstring intermediates, on the GPU."""
    for c in embedding_norm_cases:
        norm = K.embedding_ghost_norm(dev(c["ids"]), dev(c["backprops"]))
        torch.testing.assert_close(norm.cpu(), c["expected"], atol=1e-4, rtol=1e-4, msg=c["name"])
        if c["intermediates"]:
            pairs, inverse = K.embedding_unique_pairs(dev(c["ids"]))
            assert pairs.cpu().tolist() == c["intermediates"]["unique_paired_indices"]
            assert inverse.cpu().tolist() == c["intermediates"]["new_index_positions"]


# T up to 4096: lists by sorting in LDS (powers of two and their neighbours); beyond: the pairwise scan
@pytest.mark.parametrize(
    "n,T,V",
    [(1, 1, 1), (7, 10, 6), (3, 300, 50), (2, 2500, 4000), (4, 513, 3), (2, 4096, 100), (3, 2, 5), (2, 4097, 3000), (1, 9000, 7)],
)
def test_embedding_unique_pairs_bit_exact(K, n, T, V):
    torch.manual_seed(n * T)
    ids = torch.randint(0, V, (n, T))
    want_pairs, want_inv = O.embedding_unique_pairs(ids)
    pairs, inverse = K.embedding_unique_pairs(dev(ids))
    assert torch.equal(pairs.cpu(), want_pairs)
    assert torch.equal(inverse.cpu(), want_inv)


def test_embedding_unique_pairs_any_integer_ids(K):
    ids = torch.tensor([[-5, 2**40, -5, 7], [7, 7, -(2**50), 0]])
    want_pairs, want_inv = O.embedding_unique_pairs(ids)
    pairs, inverse = K.embedding_unique_pairs(dev(ids))
    assert torch.equal(pairs.cpu(), want_pairs) and torch.equal(inverse.cpu(), want_inv)


# D = 17, 1030: scalar walk; multiples of 4: the streaming norm kernel (ragged last block of rows with
# T = 40, 300); T = 4500: lists by the pairwise scan and the walking norm kernel
@pytest.mark.parametrize(
    "n,Tshape,V,D",
    [(5, (3, 2), 9, 4), (3, (40,), 7, 17), (2, (300,), 5000, 64), (2, (64,), 10, 1030), (3, (40,), 7, 1024),
     (2, (4500,), 300, 8), (2, (33, 64), 50, 260)],
)
@pytest.mark.parametrize("scale", [1.0, 5.0])
def test_embedding_grad_sample_and_norm_f32(K, n, Tshape, V, D, scale):
    torch.manual_seed(V + D)
    ids = torch.randint(0, V, (n, *Tshape))
    b = torch.randn(n, *Tshape, D)
    want = O.embedding_grad_sample(ids, b * scale, V)
    gs = K.embedding_grad_sample(dev(ids), dev(b), V, scale=scale)
    assert_rel(gs, want, FP32_REL, "embedding gs")
    # which rows are touched is integer work: exact
    assert torch.equal((gs != 0).any(dim=2).cpu(), (want != 0).any(dim=2))
    want_norm = O.embedding_norm_sample(ids, (b * scale).double())["result_sqrt"]
    norm = K.embedding_ghost_norm(dev(ids), dev(b), scale=scale)
    assert_rel(norm, want_norm, FP32_REL, "embedding norm")


def test_embedding_bf16(K):
    torch.manual_seed(5)
    ids = torch.randint(0, 11, (3, 50))
    b = torch.randn(3, 50, 24).bfloat16()
    want = O.embedding_grad_sample(ids, b.double(), 11)
    gs = K.embedding_grad_sample(dev(ids), dev(b), 11)
    assert gs.dtype == torch.bfloat16
    assert_rel(gs, want, BF16_REL)
    norm = K.embedding_ghost_norm(dev(ids), dev(b))
    assert_rel(norm, want.flatten(1).norm(dim=1), 1e-4)


@pytest.mark.parametrize("mode", ["sum", "mean"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_bag_grad_sample_is_bit_exact(K, mode, dtype):
    torch.manual_seed(17)
    V, D = 23, 10
    index = torch.randint(0, V, (40,))
    offsets = torch.tensor([0, 5, 5, 17, 18, 39])  # an empty bag, bags with repeated indices, a bag of one
    b = torch.randn(6, D).to(dtype)
    for scale in (1.0, 8.0):
        want = O.embedding_bag_grad_sample(index, offsets, (b.float() * scale).to(dtype), V, mode)
        got = K.embedding_bag_grad_sample(dev(index), dev(offsets), dev(b), V, mode=mode, scale=scale)
        assert got.dtype == dtype and torch.equal(got.cpu(), want), (mode, dtype, scale)


def test_embedding_bag_bad_inputs_raise_the_device_flag(K):
    """The entry point does not wait for the stream: a bad index writes nothing and raises a
    sticky device flag that `check_embedding_indices` reads back."""
    b = torch.ones(2, 4, device="cuda")
    K.check_embedding_indices("cuda")  # start from a clear flag
    gs = K.embedding_bag_grad_sample(dev(torch.tensor([0, 9])), dev(torch.tensor([0, 1])), b, 9)
    assert gs[0, 0].eq(1).all() and gs.sum().item() == 4.0  # bag 0 written, bag 1's index 9 dropped
    with pytest.raises(IndexError, match="outside"):
        K.check_embedding_indices("cuda")
    K.check_embedding_indices("cuda")  # cleared by the failed check
    K.embedding_bag_grad_sample(dev(torch.tensor([0, 1, 2])), dev(torch.tensor([2, 1])), b, 9)
    with pytest.raises(IndexError, match="ascending"):
        K.check_embedding_indices("cuda")
    with pytest.raises(NotImplementedError):
        K.embedding_bag_grad_sample(dev(torch.tensor([0, 1])), dev(torch.tensor([0, 1])), b, 9, mode="max")
    # a good call leaves the flag alone
    K.embedding_bag_grad_sample(dev(torch.tensor([0, 1])), dev(torch.tensor([0, 1])), b, 9)
    K.check_embedding_indices("cuda")


def test_embedding_out_of_range_id_raises_the_device_flag(K, monkeypatch):
    ids = torch.tensor([[0, 3, 9, -1]])
    b = torch.ones(1, 4, 4, device="cuda")
    K.check_embedding_indices("cuda")
    gs = K.embedding_grad_sample(dev(ids), b, 9)
    assert gs.sum().item() == 8.0 and gs[0, 0].eq(1).all() and gs[0, 3].eq(1).all()
    with pytest.raises(IndexError, match="outside"):
        K.check_embedding_indices("cuda")
    # the debugging switch checks after every call
    monkeypatch.setattr(K, "VALIDATE_EMBEDDING_INDICES", True)
    with pytest.raises(IndexError, match="outside"):
        K.embedding_grad_sample(dev(ids), b, 9)
    K.embedding_grad_sample(dev(torch.tensor([[0, 3, 8]])), b[:, :3], 9)


# ---- Normalisation layers ---------------------------------------------------------------
@pytest.mark.parametrize(
    "n,C,G,spatial",
    [
        (4, 6, 2, (3, 5)),
        (3, 64, 32, (32, 32)),  # register-resident kernel, two chunks per thread
        (2, 8, 1, (7,)),
        (2, 10, 10, (4, 4)),  # one channel per group, four chunks in all
        (2, 256, 4, ()),
        (2, 16, 2, (16, 16)),  # eight channels per group
        (2, 12, 3, (8, 8)),  # fewer chunks per channel than lanes
        (1, 32, 1, (16, 16)),  # 8192 elements: the largest register-resident group
        (1, 4, 1, (48, 48)),  # 9216 elements: streaming kernel
    ],
)
@pytest.mark.parametrize("scale", [1.0, 3.0])
def test_group_norm_grad_sample_f32(K, n, C, G, spatial, scale):
    torch.manual_seed(C + G)
    x = torch.randn(n, C, *spatial) * 2 + 0.5
    b = torch.randn(n, C, *spatial)
    want_w, want_b = O.group_norm_grad_sample(x.double(), (b * scale).double(), G, 1e-5)
    gw, gb = K.group_norm_grad_sample(dev(x), dev(b), G, 1e-5, scale=scale)
    assert_rel(gw, want_w, FP32_REL, "gn weight")
    assert_rel(gb, want_b, FP32_REL, "gn bias")
    assert_rel(gw._dpk_sumsq, want_w.pow(2).sum(1), 2e-5, "gn weight sumsq")
    assert_rel(gb._dpk_sumsq, want_b.pow(2).sum(1), 2e-5, "gn bias sumsq")


@pytest.mark.parametrize(
    "shape,D",
    [
        ((4, 8), 8),
        ((3, 5, 8), 8),
        ((2, 3, 4, 16), 16),
        ((2, 200, 260), 260),
        ((2, 130, 33), 33),
        # multiples of 256: the one-pass kernel (a row per wave in registers)
        ((2, 37, 256), 256),
        ((5, 2, 512), 512),  # fewer rows than waves
        ((3, 9, 768), 768),
        ((2, 130, 2048), 2048),
        ((1, 3, 4096), 4096),
        ((2, 5, 1280), 1280),  # a multiple of 256 without an instantiation: three-kernel path
    ],
)
def test_rms_norm_grad_sample_f32(K, shape, D):
    torch.manual_seed(D)
    x = torch.randn(*shape) + 0.3
    b = torch.randn(*shape)
    want = O.rms_norm_grad_sample(x.double(), b.double(), (D,), 1e-6)
    got = K.rms_norm_grad_sample(dev(x), dev(b), D, 1e-6)
    assert_rel(got, want, FP32_REL, "rms weight")
    # the per-sample sum of squares the kernel leaves for the optimizer's norm pass
    assert_rel(got._dpk_sumsq, want.flatten(1).pow(2).sum(1), 2e-5, "rms weight sumsq")


@pytest.mark.parametrize(
    "shape,D",
    [
        ((4, 8), 8),
        ((3, 5, 12), 12),
        ((2, 3, 4, 6), 24),  # two normalised dimensions
        ((2, 130, 33), 33),
        ((2, 37, 256), 256),  # one-pass kernel
        ((3, 9, 768), 768),
        ((2, 70, 1024), 1024),
        ((5, 2, 512), 512),
    ],
)
@pytest.mark.parametrize("scale", [1.0, 2.0])
def test_layer_norm_grad_sample_f32(K, shape, D, scale):
    torch.manual_seed(D + 1)
    x = torch.randn(*shape) * 1.5 + 0.7
    b = torch.randn(*shape)
    nshape = shape[-2:] if D == 24 else shape[-1:]
    want_w, want_b = O.layer_norm_grad_sample(x.double(), (b * scale).double(), nshape, 1e-5)
    gw, gb = K.layer_norm_grad_sample(dev(x), dev(b), D, 1e-5, scale=scale)
    assert_rel(gw._dpk_sumsq, want_w.flatten(1).pow(2).sum(1), 2e-5, "layer norm weight sumsq")
    assert_rel(gb._dpk_sumsq, want_b.flatten(1).pow(2).sum(1), 2e-5, "layer norm bias sumsq")
    assert_rel(gw, want_w.reshape(shape[0], D), FP32_REL, "ln weight")
    assert_rel(gb, want_b.reshape(shape[0], D), FP32_REL, "ln bias")
    only_w, none_b = K.layer_norm_grad_sample(dev(x), dev(b), D, 1e-5, scale=scale, want_bias=False)
    assert none_b is None
    assert_rel(only_w, want_w.reshape(shape[0], D), FP32_REL, "ln weight alone")


def test_instance_norm_is_group_norm_with_one_channel_per_group(K):
    torch.manual_seed(41)
    x, b = torch.randn(3, 5, 6, 8) + 0.3, torch.randn(3, 5, 6, 8)
    want_w, want_b = O.instance_norm_grad_sample(x.double(), b.double(), 1e-5)
    gw, gb = K.group_norm_grad_sample(dev(x), dev(b), 5, 1e-5)
    assert_rel(gw, want_w, FP32_REL)
    assert_rel(gb, want_b, FP32_REL)


def test_norm_layers_bf16(K):
    torch.manual_seed(3)
    x = torch.randn(2, 70, 64).bfloat16()
    b = torch.randn(2, 70, 64).bfloat16()
    want = O.rms_norm_grad_sample(x.double(), b.double(), (64,), 1e-6)
    assert_rel(K.rms_norm_grad_sample(dev(x), dev(b), 64, 1e-6), want, BF16_REL)
    x, b = torch.randn(3, 50, 1024).bfloat16(), torch.randn(3, 50, 1024).bfloat16()  # one-pass kernel
    want = O.rms_norm_grad_sample(x.double(), b.double(), (1024,), 1e-6)
    assert_rel(K.rms_norm_grad_sample(dev(x), dev(b), 1024, 1e-6), want, BF16_REL)
    x, b = torch.randn(3, 50, 512).bfloat16(), torch.randn(3, 50, 512).bfloat16()
    want_w, want_b = O.layer_norm_grad_sample(x.double(), b.double(), (512,), 1e-5)
    gw, gb = K.layer_norm_grad_sample(dev(x), dev(b), 512, 1e-5)
    assert_rel(gw, want_w, BF16_REL)
    assert_rel(gb, want_b, BF16_REL)
    x4, b4 = torch.randn(2, 8, 6, 6).bfloat16(), torch.randn(2, 8, 6, 6).bfloat16()
    want_w, want_b = O.group_norm_grad_sample(x4.double(), b4.double(), 4, 1e-5)
    gw, gb = K.group_norm_grad_sample(dev(x4), dev(b4), 4, 1e-5)
    assert_rel(gw, want_w, BF16_REL)
    assert_rel(gb, want_b, BF16_REL)


# ---- tied input / output embeddings: the cross term --------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
# D a multiple of 64: the tile kernel (product tile times gathered entries), ragged tiles in both
# directions, several tiles per sample, few distinct ids; other D: gather, contraction, dot product
@pytest.mark.parametrize(
    "n,T,T2,D,V",
    [(3, 7, 7, 12, 19), (2, 33, 5, 64, 300), (4, 1, 9, 8, 16), (3, 200, 150, 128, 500), (2, 300, 130, 192, 40), (9, 128, 256, 64, 1000)],
)
def test_tied_embedding_cross_term(K, dtype, n, T, T2, D, V):
    """<G_emb, G_head> against the materialised definition; embedding and projection may see
    different numbers of positions; repeated ids; the scale is a plain factor."""
    torch.manual_seed(n * 100 + T)
    ids = torch.randint(0, V, (n, T))
    if T > 2:
        ids[0, 1:3] = ids[0, 0]
    e = torch.randn(n, T, D).to(dtype)
    a = torch.randn(n, T2, D).to(dtype)
    g = (torch.randn(n, T2, V) * 0.1).to(dtype)
    _, want = O.tied_embedding_norm_sample(ids, e.double(), a.double(), g.double())
    got = K.tied_embedding_cross_term(dev(ids), dev(e), dev(a), dev(g))
    assert got.dtype == torch.float32 and got.shape == (n,)
    assert_rel(got, want, 1e-5 if dtype == torch.float32 else 1e-4, "cross term")
    assert_rel(K.tied_embedding_cross_term(dev(ids), dev(e), dev(a), dev(g), scale=4.0), 4 * want, 1e-4, "scale")
    # mixed dtypes: fp32 embedding backprops with the projection in its own dtype
    got32 = K.tied_embedding_cross_term(dev(ids), dev(e.float()), dev(a), dev(g))
    assert_rel(got32, want, 1e-4, "fp32 embedding backprops")
    assert K.tied_embedding_cross_term(dev(ids[:0]), dev(e[:0]), dev(a[:0]), dev(g[:0])).shape == (0,)
    # an id outside the table contributes nothing
    bad = ids.clone()
    bad[0, 0] = V + 3
    e0 = e.clone()
    e0[0, 0] = 0
    _, want_bad = O.tied_embedding_norm_sample(ids, e0.double(), a.double(), g.double())
    assert_rel(K.tied_embedding_cross_term(dev(bad), dev(e), dev(a), dev(g)), want_bad, 1e-5 if dtype == torch.float32 else 1e-4, "bad id")


def test_bias_grad_samples_carry_their_sumsq(K):
    """The bias entry points also return the per-sample sum of squares of what they wrote,
    so the optimizer's norm pass has nothing left to read for these tensors."""
    torch.manual_seed(9)
    b = torch.randn(7, 5, 33)
    gs = K.linear_bias_grad_sample(dev(b), scale=3.0)
    assert_rel(gs._dpk_sumsq, gs.double().pow(2).sum(1), 1e-6, "linear bias sumsq")
    assert gs._dpk_sumsq_version == gs._version
    g16 = K.linear_bias_grad_sample(dev(b.bfloat16()))
    assert_rel(g16._dpk_sumsq, g16.double().pow(2).sum(1), 1e-6, "linear bias sumsq, bf16 as stored")
    c = torch.randn(6, 9, 4, 5)
    gc = K.conv_bias_grad_sample(dev(c), scale=0.5)
    assert_rel(gc._dpk_sumsq, gc.double().pow(2).sum(1), 1e-6, "conv bias sumsq")
    gc.mul_(2.0)
    assert gc._dpk_sumsq_version != gc._version  # a write invalidates it
