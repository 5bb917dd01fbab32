"""Seeded random geometry sweeps of the Conv2d, Linear and Embedding samplers on the GPU.

The reference draws its sampler tests' shapes at random (hypothesis): Conv2d over N 0..4,
C in {1, 3, 32}, H, W 11..17, kernel 2..4, stride 1..2, padding {0, 2, "same", "valid"},
dilation 1..3, groups 1..16 (opacus/tests/grad_samples/conv2d_test.py:30-56), Linear over
2-d/3-d/4-d inputs with and without bias (linear_test.py:26-55), Embedding over 2-d/3-d/4-d id
tensors (embedding_test.py:25-61). The same spaces are drawn here with ``random.Random(0)``,
150 draws each, so that a failure names its draw; every draw calls the registered sampler of a
real ``torch.nn`` layer (the plugin boundary) on GPU tensors and compares with the CPU oracle at
the stated bars (fp32 1e-5, bf16 2e-2 with fp32 accumulation, index work exact), fp32 and bf16.
"""

import random

import pytest
import torch
import torch.nn as nn

from _compare import assert_rel
from oracle import dp_oracle as O

pytestmark = pytest.mark.gpu

FP32_REL, BF16_REL = 1e-5, 2e-2
DRAWS = 150


def expander(x):
    return 2 * x


def shrinker(x):
    return max(1, x // 2)


def conv2d_draws():
    """The reference's space; combinations it skips itself ("same" with a stride, channel counts
    the groups do not divide) are drawn again, so that all 150 draws run."""
    rng = random.Random(0)
    out = []
    while len(out) < DRAWS:
        d = dict(
            N=rng.randint(0, 4), C=rng.choice([1, 3, 32]), H=rng.randint(11, 17), W=rng.randint(11, 17),
            mapper=rng.choice([expander, shrinker]), k=rng.randint(2, 4), stride=rng.randint(1, 2),
            padding=rng.choice([0, 2, "same", "valid"]), dilation=rng.randint(1, 3), groups=rng.randint(1, 16),
        )
        d["O"] = d["mapper"](d["C"])
        if d["padding"] == "same" and d["stride"] != 1:
            continue
        if d["C"] % d["groups"] or d["O"] % d["groups"]:
            # the draw is kept with the nearest group count that divides both: most draws of 2..16
            # would otherwise be thrown away and grouped layers hardly tested
            g = d["groups"]
            while d["C"] % g or d["O"] % g:
                g -= 1
            d["groups"] = g
        out.append(d)
    # what the space holds but 150 draws may miss: groups at the maximum, "same" with dilation 3
    out.append(dict(N=3, C=32, O=16, H=13, W=16, k=3, stride=1, padding="same", dilation=3, groups=16))
    out.append(dict(N=2, C=32, O=64, H=11, W=17, k=4, stride=1, padding="same", dilation=3, groups=8))
    out.append(dict(N=4, C=32, O=64, H=17, W=11, k=2, stride=2, padding=2, dilation=2, groups=16))
    return out


CONV_DRAWS = conv2d_draws()


def _conv_id(d):
    return f"N{d['N']}-C{d['C']}-O{d['O']}-{d['H']}x{d['W']}-k{d['k']}-s{d['stride']}-p{d['padding']}-d{d['dilation']}-g{d['groups']}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_conv2d_sampler_random_geometries(dtype):
    from opacus_amd.grad_sample.conv import compute_conv_grad_sample

    assert sum(d["groups"] > 1 for d in CONV_DRAWS) > 30 and sum(d["padding"] == "same" for d in CONV_DRAWS) > 10
    for i, d in enumerate(CONV_DRAWS):
        torch.manual_seed(1000 + i)
        conv = nn.Conv2d(d["C"], d["O"], d["k"], stride=d["stride"], padding=d["padding"], dilation=d["dilation"],
                         groups=d["groups"])
        x = torch.randn(d["N"], d["C"], d["H"], d["W"]).to(dtype)
        with torch.no_grad():
            shape = conv(x.float()).shape  # the layer's own output geometry
        b = torch.randn(shape).to(dtype)
        got = compute_conv_grad_sample(conv.cuda(), [x.cuda()], b.cuda())
        what = f"draw {i} {_conv_id(d)} {dtype}"
        if d["N"] == 0:  # a batch dimension of one, all zeros (conv.py:46-53)
            assert got[conv.weight].shape == (1, *conv.weight.shape) and not got[conv.weight].any(), what
            assert got[conv.bias].shape == (1, *conv.bias.shape) and not got[conv.bias].any(), what
            continue
        k2, s2, d2 = (d["k"],) * 2, (d["stride"],) * 2, (d["dilation"],) * 2
        pad = d["padding"] if isinstance(d["padding"], str) else (d["padding"],) * 2
        want_w, want_b = O.conv2d_grad_sample(x.double(), b.double(), kernel_size=k2, padding=pad, stride=s2,
                                              dilation=d2, groups=d["groups"])
        assert got[conv.weight].shape == (d["N"], *conv.weight.shape), what
        bar = FP32_REL if dtype == torch.float32 else BF16_REL
        assert_rel(got[conv.weight], want_w, bar, what + " weight")
        assert_rel(got[conv.bias], want_b, bar, what + " bias")


def linear_draws():
    rng = random.Random(0)
    out = []
    while len(out) < DRAWS:
        d = dict(N=rng.randint(0, 4), Z=rng.randint(1, 4), H=rng.randint(1, 3), W=rng.randint(10, 17),
                 input_dim=rng.randint(2, 4), bias=rng.random() < 0.5, batch_first=rng.random() < 0.5)
        if d["input_dim"] == 2 and not d["batch_first"]:
            continue  # skipped by the reference too (linear_test.py:46-48)
        out.append(d)
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_linear_module_random_shapes(dtype):
    """Through GradSampleModule, since half the draws are not batch-first (the hooks move the
    batch dimension before the sampler sees the tensors, grad_sample_module.py:391, :413-420)."""
    import opacus_amd as A

    for i, d in enumerate(linear_draws()):
        torch.manual_seed(2000 + i)
        N, W = d["N"], d["W"]
        shape = {2: [N, W], 3: [N, d["Z"], W], 4: [N, d["Z"], d["H"], W]}[d["input_dim"]]
        lin = nn.Linear(W, W + 2, bias=d["bias"]).to(dtype)
        x = torch.randn(shape).to(dtype)
        what = f"draw {i} {d} {dtype}"
        # oracle on batch-first tensors: backprops of a sum loss are the loss's gradient at the output
        w_out = torch.randn(*shape[:-1], W + 2).to(dtype)
        want_w, want_b = O.linear_grad_sample(x.double(), w_out.double(), bias=d["bias"])
        xin, wout = (x, w_out) if d["batch_first"] else (x.transpose(0, 1), w_out.transpose(0, 1))
        gsm = A.GradSampleModule(lin.cuda(), batch_first=d["batch_first"], loss_reduction="sum")
        out = gsm(xin.cuda())
        (out * wout.cuda()).sum().backward()
        bar = FP32_REL if dtype == torch.float32 else BF16_REL
        if N == 0:
            assert lin.weight.grad_sample.shape[0] == 0, what
        else:
            assert lin.weight.grad_sample.shape == (N, W + 2, W), what
            assert_rel(lin.weight.grad_sample, want_w, bar, what + " weight")
            if d["bias"]:
                assert_rel(lin.bias.grad_sample, want_b, bar, what + " bias")
        gsm.to_standard_module()


def embedding_draws():
    rng = random.Random(0)
    return [
        dict(N=rng.randint(0, 4), T=rng.randint(1, 5), Q=rng.randint(1, 4), R=rng.randint(1, 2), V=rng.randint(2, 32),
             D=rng.randint(10, 17), dim=rng.randint(2, 4), batch_first=rng.random() < 0.5)
        for _ in range(DRAWS)
    ]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_embedding_module_random_shapes(dtype):
    import opacus_amd as A
    from opacus_amd import kernels

    kernels.check_embedding_indices("cuda")
    for i, d in enumerate(embedding_draws()):
        torch.manual_seed(3000 + i)
        N, V, D = d["N"], d["V"], d["D"]
        size = {2: [N, d["T"]], 3: [N, d["T"], d["Q"]], 4: [N, d["T"], d["Q"], d["R"]]}[d["dim"]]
        emb = nn.Embedding(V, D).to(dtype)
        ids = torch.randint(0, V, size)
        w_out = torch.randn(*size, D).to(dtype)
        what = f"draw {i} {d} {dtype}"
        xin, wout = (ids, w_out) if d["batch_first"] else (ids.transpose(0, 1), w_out.transpose(0, 1))
        gsm = A.GradSampleModule(emb.cuda(), batch_first=d["batch_first"], loss_reduction="sum")
        (gsm(xin.cuda()) * wout.cuda()).sum().backward()
        gs = emb.weight.grad_sample
        if N == 0:
            # the sampler returns zeros with a batch dimension of one (embedding.py:44-46); stored into the
            # hooks' buffer of max_batch_len = 0 rows that is an empty tensor (grad_sample_module.py:61-66)
            assert gs.shape == (0, V, D), what
            from opacus_amd.grad_sample.embedding import compute_embedding_grad_sample

            direct = compute_embedding_grad_sample(emb, [ids.cuda()], w_out.cuda())[emb.weight]
            assert direct.shape == (1, V, D) and not direct.any(), what
        else:
            want = O.embedding_grad_sample(ids, w_out.double(), V)
            assert gs.shape == (N, V, D), what
            assert_rel(gs, want, FP32_REL if dtype == torch.float32 else BF16_REL, what)
            # which rows of the table a sample touches is index work: exact
            touched = torch.zeros(N, V, dtype=torch.bool)
            touched.scatter_(1, ids.reshape(N, -1), True)
            assert not (gs.cpu()[~touched] != 0).any(), what + ": a row no id names was written"
            # and the ghost norm of the same draw
            norm = kernels.embedding_ghost_norm(ids.cuda(), w_out.cuda())
            assert_rel(norm, want.flatten(1).norm(dim=1), 1e-5 if dtype == torch.float32 else 1e-4, what + " ghost norm")
        gsm.to_standard_module()
    kernels.check_embedding_indices("cuda")  # no id was out of range
