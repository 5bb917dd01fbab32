"""DP-SGD step throughput on one MI355X: ``python bench.py --gpus 1 --steps K --warmup W``.

Default workload (the one the headline metric is quoted on, ``--workload c2``): a single
``nn.Linear(4096, 4096, bias=True)`` in fp32, batch 128, one position per sample, hooks
mode: forward, backward (per-sample gradients, 128 x 4096 x 4096 fp32 = 8.59 GB), then
``DPOptimizer.step`` (clip at C = 1, accumulate, noise sigma = 1, SGD update) and
``zero_grad``. Inputs are synthetic tensors resident in HBM before the clock starts.

Prints ONE JSON line. ``roofline`` describes the dominant kernel of the step, timed with
HIP events on the launch stream inside the timed region. ``cpu_baseline`` is the CPU
oracle - a restatement of the reference's einsum path, allocation pattern included -
timed on this box's host cores on a bounded sample of the same workload.

The headline fields are config 2's. The same run then times the other four benchmark
configurations (c1, c3, c4, c5: full DP-SGD steps through the drop-in API, at most 20
steps each, 10 for c5) and reports them under ``"configs"``, each with its own
``ms_per_step``, ``samples_per_s``, ``roofline`` and bounded-sample ``cpu_baseline``.
Beside every configuration (the headline included) ``plain_step`` is the same model, batch and
loss without any DP wrapper (forward + backward + SGD), timed in the same process with the same
loop, and ``dp_over_plain`` the ratio of the two step times
(c5 also with embedding table and LM head tied, which the reference refuses under ghost
clipping, as ``tied_embeddings``).
``--workload cN`` times one configuration alone (same JSON shape, no ``configs``);
``--headline-only`` skips the other four. ``--kernels`` times each kernel of the library on
its own at those shapes and prints one JSON line per kernel (time, algorithmic work,
fraction of its roofline).
"""

from __future__ import annotations

import argparse
import copy
import json
import os
import sys
import time
import warnings
from pathlib import Path

import torch
import torch.nn as nn
import torch.nn.functional as F

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

# MI355X published peaks
HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
MFMA_FP32_PEAK_TFLOPS = 157.3


# ---- models of the five configurations -------------------------------------------------
class SmallCNN(nn.Module):
    def __init__(self):
        super().__init__()
        self.conv1 = nn.Conv2d(1, 16, 8, 2, padding=3)
        self.conv2 = nn.Conv2d(16, 32, 4, 2)
        self.fc1 = nn.Linear(32 * 4 * 4, 32)
        self.fc2 = nn.Linear(32, 10)

    def forward(self, x):
        x = F.max_pool2d(F.relu(self.conv1(x)), 2, 1)
        x = F.max_pool2d(F.relu(self.conv2(x)), 2, 1)
        return self.fc2(F.relu(self.fc1(x.flatten(1))))


class ResBlock(nn.Module):
    def __init__(self, ch=64, groups=32):
        super().__init__()
        self.c1, self.g1 = nn.Conv2d(ch, ch, 3, padding=1), nn.GroupNorm(groups, ch)
        self.c2, self.g2 = nn.Conv2d(ch, ch, 3, padding=1), nn.GroupNorm(groups, ch)
        self.head = nn.Linear(ch, 10)

    def forward(self, x):
        h = F.relu(self.g1(self.c1(x)))
        h = F.relu(self.g2(self.c2(h)) + x)
        return self.head(h.mean(dim=(2, 3)))


class Llama(nn.Module):
    """Decoder stack: RMSNorm, grouped-query attention with rotary embedding, SwiGLU;
    bias-free. ``tied=False`` keeps embedding and LM head apart, which is what the reference
    can run (it refuses tied parameters under ghost clipping); ``tied=True`` shares the table."""

    def __init__(self, vocab=32000, d=2048, heads=16, kv=4, ffn=5632, layers=4, tied=False):
        super().__init__()
        self.emb = nn.Embedding(vocab, d)
        self.heads, self.kv, self.hd = heads, kv, d // heads
        self.blocks = nn.ModuleList(
            nn.ModuleDict(
                dict(
                    n1=nn.RMSNorm(d, eps=1e-5),
                    q=nn.Linear(d, d, bias=False),
                    k=nn.Linear(d, kv * (d // heads), bias=False),
                    v=nn.Linear(d, kv * (d // heads), bias=False),
                    o=nn.Linear(d, d, bias=False),
                    n2=nn.RMSNorm(d, eps=1e-5),
                    gate=nn.Linear(d, ffn, bias=False),
                    up=nn.Linear(d, ffn, bias=False),
                    down=nn.Linear(ffn, d, bias=False),
                )
            )
            for _ in range(layers)
        )
        self.norm = nn.RMSNorm(d, eps=1e-5)
        self.lm_head = nn.Linear(d, vocab, bias=False)
        if tied:
            self.lm_head.weight = self.emb.weight

    @staticmethod
    def rope(x):
        T, D = x.shape[-2], x.shape[-1]
        pos = torch.arange(T, device=x.device, dtype=torch.float32)
        inv = 1.0 / (10000 ** (torch.arange(0, D, 2, device=x.device, dtype=torch.float32) / D))
        ang = pos[:, None] * inv[None, :]
        cos, sin = ang.cos().to(x.dtype), ang.sin().to(x.dtype)
        x1, x2 = x[..., 0::2], x[..., 1::2]
        return torch.stack([x1 * cos - x2 * sin, x1 * sin + x2 * cos], dim=-1).flatten(-2)

    def forward(self, ids):
        h = self.emb(ids)
        B, T, _ = h.shape
        for blk in self.blocks:
            a = blk["n1"](h)
            q = blk["q"](a).view(B, T, self.heads, self.hd).transpose(1, 2)
            k = blk["k"](a).view(B, T, self.kv, self.hd).transpose(1, 2)
            v = blk["v"](a).view(B, T, self.kv, self.hd).transpose(1, 2)
            q, k = self.rope(q), self.rope(k)
            att = F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
            h = h + blk["o"](att.transpose(1, 2).reshape(B, T, -1))
            m = blk["n2"](h)
            h = h + blk["down"](F.silu(blk["gate"](m)) * blk["up"](m))
        return self.lm_head(self.norm(h))


class PerSampleMSE(nn.Module):
    """Mean squared error against zeros, one value per sample (mean over positions and features)."""

    def __init__(self, reduction="mean"):
        super().__init__()
        self.reduction = reduction

    def forward(self, out, _target=None):
        l = out.float().pow(2).flatten(1).mean(1)
        if self.reduction == "none":
            return l
        return l.mean() if self.reduction == "mean" else l.sum()


def ghost_executed_flops(model: nn.Module, n: int, T: int) -> float:
    """MFMA FLOPs the ghost-norm entry point executes per step over the (bf16) Linear layers:
    128 x 128 tiles of the upper block-triangle of both Gram matrices, or, for a layer thin
    enough that forming its gradient tiles is cheaper (the library's rule, repeated here), the
    contraction over T itself."""
    nt = (T + 127) // 128
    pairs = nt * (nt + 1) // 2
    total = 0.0
    for m in model.modules():
        if isinstance(m, nn.Linear):
            gram = pairs * 128.0 * 128 * (m.in_features + m.out_features)
            direct = float(T) * m.in_features * m.out_features
            total += n * 2.0 * (direct if T > 1 and direct < 0.9 * gram else gram)
    return total


# ---- workloads ----------------------------------------------------------------------------
def workload_c2(dev, lazy=False):
    """``lazy=True``: the library's opt-in ``lazy_linear_grad_sample`` (the weight's per-sample gradient
    is kept as activations and backprops; norms from the closed form, clipped sum from one weighted
    contraction, the 8.6 GB tensor formed only if somebody reads it). Never the headline."""
    from opacus_amd import GradSampleModule
    from opacus_amd.optimizers import DPOptimizer

    N, D_IN, D_OUT = 128, 4096, 4096
    torch.manual_seed(0)
    lin = nn.Linear(D_IN, D_OUT, bias=True)
    x, b = torch.randn(N, D_IN).to(dev), torch.randn(N, D_OUT).to(dev)
    model = GradSampleModule(lin.to(dev), loss_reduction="sum", lazy_linear_grad_sample=lazy)
    opt = DPOptimizer(
        torch.optim.SGD(model.parameters(), lr=0.05), noise_multiplier=1.0, max_grad_norm=1.0,
        expected_batch_size=N, loss_reduction="sum",
    )

    def step():
        opt.zero_grad(set_to_none=True)
        model(x).backward(b)  # backprops ~ N(0,1) injected at the layer output
        opt.step()

    def plain():
        torch.manual_seed(0)
        ref = nn.Linear(D_IN, D_OUT, bias=True).to(dev)
        sgd = torch.optim.SGD(ref.parameters(), lr=0.05)

        def plain_step():
            sgd.zero_grad(set_to_none=True)
            ref(x).backward(b)
            sgd.step()

        return plain_step

    P = D_OUT * D_IN + D_OUT
    if lazy:
        return dict(
            step=step, plain=plain, n=N, dtype="f32",
            workload="Linear(4096->4096, bias) fp32, batch 128, T=1, hooks with lazy_linear_grad_sample=True: norms from the "
                     "closed form, clipped sum from one weighted contraction, grad_sample never read so never formed",
            extra={"lazy_linear_grad_sample": True},
            roofline=dict(
                kernel="linear_wsum_generic_kernel<128,128,float,float> (clipped sum of the weight: one fp32 MFMA contraction "
                       "over the 128 rows, coefficients on the rows of the backprops)",
                timer="linear_weighted_sum", bound="mfma", work_per_launch=2.0 * N * D_IN * D_OUT, unit="TFLOP/s",
                peak=MFMA_FP32_PEAK_TFLOPS, traffic=None),
        )
    return dict(
        step=step, plain=plain, n=N, dtype="f32",
        workload="Linear(4096->4096, bias) fp32, batch 128, T=1, hooks per-sample grad + clip(C=1) + noise(sigma=1) + SGD",
        extra={"per_sample_grad_bytes": N * P * 4},
        # one call covers weight and bias: reads n * P * 4 bytes, writes P * 4 bytes. The timed span
        # holds two dispatches: the wide kernel on the 512 whole 128 KB spans of the weight and the
        # one-wave kernel on the 4096 bias columns (a few microseconds).
        roofline=dict(
            kernel="clip_accumulate_wide_kernel<float,float> (+ clip_accumulate_kernel on the bias, same call)",
            timer="clip_accumulate",
            bound="hbm", work_per_launch=float(N * P * 4 + P * 4), unit="GB/s", peak=HBM_PEAK_GBS,
            # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE (KiB per
            # dispatch), each scaled by what the counter reads for a 1 GiB device copy
            # (FETCH_SIZE x 2.000, WRITE_SIZE x 1.000): 8,390,265 + 65,551 KiB over the two dispatches.
            traffic=8455816 * 1024,
            traffic_source="recorded: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command, "
                           "profiles/clip_accumulate_linear4096_b128_hbm_traffic.txt (not re-measured by this run)",
        ),
    )


def _hooks_workload(dev, net, x, y, n, sigma, desc, roofline, dtype="f32", autograd_weight_grads=False):
    """``autograd_weight_grads=False``: the library's option under which backward() forms no
    aggregate (non-private) weight gradients, which the DP step never reads; the default of the
    library keeps them as the reference does (workloads c1d / c4d)."""
    from opacus_amd import GradSampleModule
    from opacus_amd.optimizers import DPOptimizer

    plain_net = copy.deepcopy(net)
    model = GradSampleModule(net.to(dev), loss_reduction="mean", autograd_weight_grads=autograd_weight_grads)
    desc += "" if autograd_weight_grads else ", autograd_weight_grads=False"
    opt = DPOptimizer(
        torch.optim.SGD(model.parameters(), lr=0.1), noise_multiplier=sigma, max_grad_norm=1.0, expected_batch_size=n
    )
    x, y = x.to(dev), y.to(dev)

    def step():
        opt.zero_grad(set_to_none=True)
        F.cross_entropy(model(x), y).backward()
        opt.step()

    def plain():
        ref = plain_net.to(dev)
        sgd = torch.optim.SGD(ref.parameters(), lr=0.1)

        def plain_step():
            sgd.zero_grad(set_to_none=True)
            F.cross_entropy(ref(x), y).backward()
            sgd.step()

        return plain_step

    return dict(step=step, plain=plain, n=n, dtype=dtype, workload=desc, extra={"autograd_weight_grads": autograd_weight_grads},
                roofline=roofline)


def workload_c1(dev, autograd_weight_grads=False):
    torch.manual_seed(0)
    n = 256
    P = 26010
    return _hooks_workload(
        dev, SmallCNN(), torch.randn(n, 1, 28, 28), torch.randint(0, 10, (n,)), n, 1.1,
        "Small CNN (conv 1->16 k8 s2 p3, conv 16->32 k4 s2, fc 512->32, fc 32->10) fp32, batch 256, hooks, C=1, sigma=1.1",
        # the optimizer's whole step on the eight parameter tensors as one launch: reads every per-sample
        # gradient once (n*P*4), writes the noised gradient and the clipped sum (2*P*4)
        dict(kernel="clip_noise_step_kernel<float,float> (clip factors, clipped sum, noise and scaling of all 8 tensors, one launch)",
             timer="clip_noise_step", bound="hbm", work_per_launch=float(n * P * 4 + 2 * P * 4), unit="GB/s", peak=HBM_PEAK_GBS,
             traffic=26995456,
             traffic_source="recorded: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of bench.py --workload c1, profiles/clip_noise_step_small_cnn_b256_hbm_traffic.txt (not re-measured by this run)"),
        autograd_weight_grads=autograd_weight_grads,
    )


def workload_c4(dev, autograd_weight_grads=False):
    torch.manual_seed(0)
    n = 256
    flops = 2.0 * n * 64 * 576 * 1024  # per conv launch
    return _hooks_workload(
        dev, ResBlock(), torch.randn(n, 64, 32, 32), torch.randint(0, 10, (n,)), n, 1.0,
        "ResNet basic block: 2 x Conv2d(64->64, 3x3, p1) + GroupNorm(32), 32x32 images, fp32, batch 256, hooks, C=1, sigma=1",
        dict(kernel="conv2d_gs_patch_kernel<64,64,float,float>", timer="conv2d_gs", bound="mfma",
             work_per_launch=flops, unit="TFLOP/s", peak=MFMA_FP32_PEAK_TFLOPS,
             # inputs 134.2 MB + per-sample gradients 37.7 MB = 172.0 MB must move once
             traffic=174340597,
             traffic_source="recorded: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of bench.py --workload c4, profiles/conv2d_gs_resblock_b256_hbm_traffic.txt (not re-measured by this run)"),
        autograd_weight_grads=autograd_weight_grads,
    )


def _ghost_workload(dev, net, make_inputs, loss_call, n, T, sigma, desc, single=True, traffic=None, traffic_source=None,
                    wsum_traffic=None, wsum_traffic_source=None, plain_loss=None):
    from opacus_amd import GradSampleModuleFastGradientClipping
    from opacus_amd.optimizers import DPOptimizerFastGradientClipping

    plain_net = copy.deepcopy(net)
    net = net.to(dev).bfloat16()
    model = GradSampleModuleFastGradientClipping(net, loss_reduction="mean", max_grad_norm=1.0, single_backward=single)
    opt = DPOptimizerFastGradientClipping(
        torch.optim.SGD(model.parameters(), lr=0.01), noise_multiplier=sigma, max_grad_norm=1.0, expected_batch_size=n
    )
    inputs = make_inputs()

    def step():
        opt.zero_grad(set_to_none=True)
        loss_call(model, opt, inputs).backward()
        opt.step()

    def plain():
        ref = plain_net.to(dev).bfloat16()
        sgd = torch.optim.SGD(ref.parameters(), lr=0.01)

        def plain_step():
            sgd.zero_grad(set_to_none=True)
            plain_loss(ref, inputs).backward()
            sgd.step()

        return plain_step

    flops = ghost_executed_flops(net, n, T)
    ghost = dict(kernel="ghost_norm_multi_kernel<128x128, 2 stages> (all Linear layers of a step pooled into one launch, the units "
                        "past the last whole round of resident blocks each cut into four pieces along the contraction; thin layers "
                        "by linear_dlds_kernel; ghost_norm_bf16_dlds_kernel layer by layer with two backward passes)",
                 timer="linear_ghost_norm", bound="mfma", work_per_step=flops, unit="TFLOP/s",
                 peak=MFMA_BF16_PEAK_TFLOPS, traffic=traffic, **({"traffic_source": traffic_source} if traffic else {}))
    out = dict(
        step=step, plain=plain, n=n, dtype="bf16", workload=desc + (", one backward pass (library default)" if single else ", two backward passes (single_backward=False)"),
        extra={"ghost_norm_executed_flops_per_step": flops, "single_backward": single},
        roofline=ghost,
    )
    if single:
        # with one backward pass the clipped sums are this library's kernel too, and the longer of the two
        wsum_flops = sum(2.0 * n * T * m.in_features * m.out_features for m in net.modules() if isinstance(m, nn.Linear))
        out["roofline"] = dict(
            kernel="linear_wsum_multi_kernel<256x256> (clip-weighted sums of all Linear layers in one pooled launch; a pool "
                   "with fewer tiles than resident blocks is cut into pieces of samples whose fp32 partial sums "
                   "add_pieces_multi_kernel adds, and the time covers both kernels)",
            timer="linear_weighted_sum", bound="mfma", work_per_step=wsum_flops, unit="TFLOP/s", peak=MFMA_BF16_PEAK_TFLOPS,
            traffic=wsum_traffic, **({"traffic_source": wsum_traffic_source} if wsum_traffic else {}))
        out["roofline_also"] = {"roofline_ghost_norm": ghost}
        out["extra"]["weighted_sum_flops_per_step"] = wsum_flops
    return out


def workload_c3(dev, single=True):
    from opacus_amd import DPLossFastGradientClipping

    torch.manual_seed(0)
    n, T = 32, 512
    net = nn.Sequential(nn.Linear(1024, 4096), nn.GELU(), nn.Linear(4096, 1024))
    crit = {}

    def loss_call(model, opt, x):
        if "c" not in crit:
            crit["c"] = DPLossFastGradientClipping(model, opt, PerSampleMSE("mean"), "mean")
        return crit["c"](model(x), None)

    return _ghost_workload(
        dev, net, lambda: torch.randn(n, T, 1024).to(dev).bfloat16(), loss_call, n, T, 1.0,
        "MLP Linear(1024->4096) GELU Linear(4096->1024), bf16, batch 32, T=512, ghost clipping, C=1, sigma=1",
        single=single, plain_loss=lambda ref, x: PerSampleMSE("mean")(ref(x)),
        # HBM bytes of the pooled launch (operands of both layers: 335.5 MB must be read once)
        traffic=367228187 if single else None,
        traffic_source="recorded: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of bench.py --workload c3, profiles/ghost_norm_multi_mlp_b32_t512_hbm_traffic.txt (not re-measured by this run)",
        # the pooled launch and the kernel that adds its pieces: 335.5 MB of operands read once, 67.1 MB of
        # fp32 piece sums written and read again, 16.8 MB of bf16 results written
        wsum_traffic=553920016,
        wsum_traffic_source="recorded: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of bench.py --workload c3, profiles/weighted_sum_multi_mlp_b32_t512_hbm_traffic.txt (not re-measured by this run)",
    )


def workload_c5(dev, tied=False, single=True):
    from opacus_amd import DPLossFastGradientClipping

    torch.manual_seed(0)
    n, T, V = 16, 1024, 32000
    net = Llama(tied=tied)
    crit = {}

    def loss_call(model, opt, ids):
        if "c" not in crit:
            crit["c"] = DPLossFastGradientClipping(model, opt, nn.CrossEntropyLoss(), "mean")
        logits = model(ids)[:, :-1]
        return crit["c"](logits.reshape(-1, V).float(), ids[:, 1:].reshape(-1), shape=(n, T - 1, V))

    return _ghost_workload(
        dev, net, lambda: torch.randint(0, V, (n, T)).to(dev), loss_call, n, T, 0.8,
        f"4-layer Llama-style decoder (d 2048, 16 heads / 4 KV, SwiGLU 5632, vocab 32000, {'tied' if tied else 'untied'}), "
        "bf16, batch 16, seq 1024, ghost clipping, C=1, sigma=0.8",
        single=single,
        plain_loss=lambda ref, ids: F.cross_entropy(ref(ids)[:, :-1].reshape(-1, V).float(), ids[:, 1:].reshape(-1)),
        # HBM bytes of the pooled launch (21 layers by the Gram route; their operands, 5.21 GB, must be
        # read once; a unit streams two 128-row blocks of both operands and the 4 MB L2 of an XCD does not
        # hold a sample's rows of the wide layers, so the units re-fetch from the last-level cache)
        traffic=11340730370 if single and not tied else None,
        traffic_source="recorded: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of bench.py --workload c5, "
                       "profiles/ghost_norm_multi_llama_b16_t1024_hbm_traffic.txt (not re-measured by this run)",
        # the pooled launch: 5.88 GB of operands and 0.49 GB of results must move once; a tile streams 256
        # columns of both operands over all 16384 rows, and the narrow operand of a layer (67 MB, which
        # stays in the 256 MB last-level cache) is fetched again by every row of tiles
        wsum_traffic=14199424257 if not tied else None,
        wsum_traffic_source="recorded: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of bench.py --workload c5, "
                            "profiles/weighted_sum_multi_llama_b16_t1024_hbm_traffic.txt (not re-measured by this run)",
    )


def workload_c5_tied(dev):
    return workload_c5(dev, tied=True)


WORKLOADS = {
    "c1": workload_c1, "c2": workload_c2, "c3": workload_c3, "c4": workload_c4, "c5": workload_c5,
    "c5t": workload_c5_tied,
    # the same two with the reference's two backward passes (single_backward=False)
    "c3p": lambda dev: workload_c3(dev, single=False), "c5p": lambda dev: workload_c5(dev, single=False),
    # c1 and c4 with the library's default hooks (autograd's own weight gradients kept, as in the reference)
    # c2 with the opt-in lazy per-sample gradient of the Linear weight (reported beside the headline only)
    "c2l": lambda dev: workload_c2(dev, lazy=True),
    "c1d": lambda dev: workload_c1(dev, autograd_weight_grads=True),
    "c4d": lambda dev: workload_c4(dev, autograd_weight_grads=True),
}


# ---- CPU baselines: the oracle's restatement of the reference's step on the host cores ----------
warnings.filterwarnings("ignore", message="Full backward hook is firing")  # layers at the graph's start


def _cpu_capture(net):
    """Forward / backward hooks of plain torch that keep each sampled layer's input and output
    gradient, as the reference's hooks do (grad_sample_module.py:291-365)."""
    store, handles = {}, []
    kinds = (nn.Linear, nn.Conv2d, nn.GroupNorm, nn.RMSNorm, nn.Embedding)
    for m in net.modules():
        if isinstance(m, kinds):
            handles.append(m.register_forward_hook(lambda mod, inp, out: store.setdefault(mod, [None, None]).__setitem__(0, inp[0].detach())))
            handles.append(m.register_full_backward_hook(lambda mod, gi, go: store[mod].__setitem__(1, go[0].detach())))
    return store, handles


def _cpu_grad_samples(O, m, a, b):
    """Per-sample gradients of one layer's own parameters, in ``m.parameters()`` order."""
    if isinstance(m, nn.Linear):
        gw, gb = O.linear_grad_sample(a, b, bias=m.bias is not None)
    elif isinstance(m, nn.Conv2d):
        gw, gb = O.conv2d_grad_sample(a, b, kernel_size=m.kernel_size, padding=m.padding, stride=m.stride,
                                      dilation=m.dilation, groups=m.groups, bias=m.bias is not None)
    elif isinstance(m, nn.GroupNorm):
        gw, gb = O.group_norm_grad_sample(a, b, m.num_groups, m.eps)
    elif isinstance(m, nn.RMSNorm):
        gw, gb = O.rms_norm_grad_sample(a, b, m.normalized_shape, m.eps), None
    else:
        gw, gb = O.embedding_grad_sample(a, b, m.num_embeddings), None
    return [g for g in (gw, gb) if g is not None]


def _cpu_hooks_step(O, net, sgd, x, y, n, sigma, C=1.0):
    """One step in hooks mode: autograd's backward, every layer's einsum sampler, the zero +
    copy buffer, norms, clip, sum, noise, scale, SGD (the reference's passes, one by one)."""
    store, handles = _cpu_capture(net)
    sgd.zero_grad(set_to_none=True)
    F.cross_entropy(net(x), y).backward()
    for h in handles:
        h.remove()
    gs, params = [], []
    for m, (a, b) in store.items():
        b = O.scale_backprops(b, n, "mean")
        for g in _cpu_grad_samples(O, m, a, b):
            gs.append(O.store_grad_sample(g, n))
        params += list(m.parameters(recurse=False))
    _, _, summed = O.clip_and_accumulate(gs, C)
    grads = O.add_noise_and_scale(summed, [p.shape for p in params], sigma, C, n, "mean")
    for p, g in zip(params, grads):
        p.grad = g
    sgd.step()


def _cpu_ghost_step(O, net, sgd, inputs, per_sample_loss, n, sigma, C=1.0):
    """One ghost-clipping step: first backward with the norm samplers (Gram products for Linear,
    index sums for Embedding, materialised gradients for RMSNorm), clipping coefficients, second
    backward of the reweighted loss, noise, scale, SGD (fast_gradient_clipping_utils.py:179-203)."""
    store, handles = _cpu_capture(net)
    sgd.zero_grad(set_to_none=True)
    losses = per_sample_loss(net(inputs))
    losses.mean().backward(retain_graph=True)
    for h in handles:
        h.remove()
    norms = []
    for m, (a, b) in store.items():
        b = O.scale_backprops(b, n, "mean")
        if isinstance(m, nn.Linear):
            nw, nb = O.linear_norm_sample(a, b, bias=m.bias is not None)
            norms += [v.float() for v in (nw, nb) if v is not None]
        elif isinstance(m, nn.Embedding):
            norms.append(O.embedding_norm_sample(a, b)["result_sqrt"].float())
        else:
            norms += [g.flatten(1).norm(2, dim=1).float() for g in _cpu_grad_samples(O, m, a, b)]
    coef = O.clipping_coef(norms, C)
    sgd.zero_grad(set_to_none=True)
    (coef * losses).sum().backward()
    params = [p for p in net.parameters() if p.grad is not None]
    grads = O.add_noise_and_scale([p.grad for p in params], [p.shape for p in params], sigma, C, n, "mean")
    for p, g in zip(params, grads):
        p.grad = g.to(p.dtype)
    sgd.step()


def _cpu_time(step, n_sample, n_full, steps, what, warm=True):
    if warm:
        step()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    dt = time.perf_counter() - t0
    return {
        "value": n_sample * steps / dt,
        "unit": "samples/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{steps} step(s) at batch {n_sample} of {n_full}{' after one warm-up step' if warm else ', no warm-up'} ({what}; every per-sample "
                  f"pass is linear in the batch); {os.cpu_count()} logical CPUs visible",
    }


def cpu_baseline(workload: str = "c2") -> dict:
    """The oracle's DP-SGD step for ``workload`` on the host cores, on a bounded sample of its batch."""
    from oracle import dp_oracle as O

    torch.manual_seed(0)
    if workload == "c2":
        N, D_IN, D_OUT, n_sample = 128, 4096, 4096, 16
        lin = nn.Linear(D_IN, D_OUT, bias=True)
        x, b = torch.randn(n_sample, D_IN), torch.randn(n_sample, D_OUT)
        sgd = torch.optim.SGD(lin.parameters(), lr=0.05)

        def step():
            sgd.zero_grad(set_to_none=True)
            lin(x).backward(b)
            bp = O.scale_backprops(b, n_sample, "sum")
            gs_w, gs_b = O.linear_grad_sample(x, bp)
            gs = [O.store_grad_sample(gs_w, n_sample), O.store_grad_sample(gs_b, n_sample)]
            _, _, summed = O.clip_and_accumulate(gs, 1.0)
            grads = O.add_noise_and_scale(summed, [lin.weight.shape, lin.bias.shape], 1.0, 1.0, n_sample, "sum")
            lin.weight.grad, lin.bias.grad = grads
            sgd.step()

        return _cpu_time(step, n_sample, N, 3, "einsum sampler, zero + copy buffer, norms, clip, sum, noise")
    if workload in ("c1", "c4"):
        if workload == "c1":
            net, N, n_sample, steps = SmallCNN(), 256, 256, 10
            x, sigma = torch.randn(n_sample, 1, 28, 28), 1.1
        else:
            net, N, n_sample, steps = ResBlock(), 256, 64, 3
            x, sigma = torch.randn(n_sample, 64, 32, 32), 1.0
        y = torch.randint(0, 10, (n_sample,))
        sgd = torch.optim.SGD(net.parameters(), lr=0.1)
        return _cpu_time(lambda: _cpu_hooks_step(O, net, sgd, x, y, n_sample, sigma), n_sample, N, steps,
                         "hooks mode: unfold + einsum samplers, zero + copy buffers, norms, clip, sum, noise")
    if workload == "c3":
        N, n_sample, T = 32, 8, 512
        net = nn.Sequential(nn.Linear(1024, 4096), nn.GELU(), nn.Linear(4096, 1024)).bfloat16()
        x = torch.randn(n_sample, T, 1024).bfloat16()
        sgd = torch.optim.SGD(net.parameters(), lr=0.01)
        loss = lambda out: out.float().pow(2).flatten(1).mean(1)  # noqa: E731
        return _cpu_time(lambda: _cpu_ghost_step(O, net, sgd, x, loss, n_sample, 1.0), n_sample, N, 3,
                         "ghost clipping in bf16: T x T Gram norm samplers, two backward passes, noise")
    if workload == "c5":
        N, n_sample, T, V = 16, 1, 1024, 32000
        net = Llama().bfloat16()
        ids = torch.randint(0, V, (n_sample, T))
        sgd = torch.optim.SGD(net.parameters(), lr=0.01)

        def loss(logits):
            tok = F.cross_entropy(logits[:, :-1].reshape(-1, V).float(), ids[:, 1:].reshape(-1), reduction="none")
            return tok.view(n_sample, T - 1).mean(1)

        return _cpu_time(lambda: _cpu_ghost_step(O, net, sgd, ids, loss, n_sample, 0.8), n_sample, N, 1,
                         "ghost clipping in bf16: Gram, embedding and RMSNorm norm samplers, two backward passes, noise",
                         warm=False)
    raise ValueError(workload)


def kernel_table(dev, iters: int = 10, warm: int = 3, with_cpu: bool = True):
    """Every kernel of the library on its own at the benchmark configurations' shapes: yields one
    dict per kernel with its time (HIP events on the launch stream) against the roofline that
    bounds it. Work figures are algorithmic: bytes that must cross HBM once, or executed MFMA
    FLOPs (the ghost-norm kernels visit the block-triangle of the T x T Gram)."""
    from opacus_amd import kernels as K

    if with_cpu:
        from oracle import dp_oracle as O

    def timed(fn):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(iters):
            fn()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / iters

    def cpu(fn, factor, sample):
        """The CPU oracle's function for the same row on a bounded sample of the batch, scaled
        linearly (every one of these passes is linear in the number of samples)."""
        if not with_cpu:
            return None
        fn()
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        return {"ms": dt * 1e3 * factor, "kind": "port", "cores": torch.get_num_threads(),
                "sample": f"{sample}, time x {factor:g}"}

    def row(name, ref_row, shape, ms, bound, work, cpu_baseline=None):
        peak, unit, scale = {
            "hbm": (HBM_PEAK_GBS, "GB/s", 1e9),
            "mfma_bf16": (MFMA_BF16_PEAK_TFLOPS, "TFLOP/s", 1e12),
            "mfma_fp32": (MFMA_FP32_PEAK_TFLOPS, "TFLOP/s", 1e12),
        }[bound]
        ach = work / (ms * 1e-3) / scale
        out = {"kernel": name, "row": ref_row, "shape": shape, "ms": ms, "bound": bound, "achieved": ach,
               "peak": peak, "unit": unit, "frac": ach / peak, "algorithmic_work": work}
        if cpu_baseline is not None:
            out["cpu_baseline"] = cpu_baseline
        return out

    def tri_tiles(T, tile=128):
        nt = -(-T // tile)
        return nt * (nt + 1) // 2, nt * nt

    torch.manual_seed(0)
    # ---- C2: Linear 4096x4096 fp32, batch 128, T = 1
    n, d = 128, 4096
    a, b = torch.randn(n, d, device=dev), torch.randn(n, d, device=dev)
    gs, ss = K.linear_grad_sample(b, a)
    ca, cb = a[:8].cpu(), b[:8].cpu()
    yield row("linear_gs (T=1 outer product)", "a1", "C2 n=128 4096x4096 f32", timed(lambda: K.linear_grad_sample(b, a)),
              "hbm", gs.numel() * 4 + 2 * n * d * 4,
              cpu(lambda: O.store_grad_sample(O.linear_grad_sample(ca, cb)[0], 8), 16, "8 of 128 samples, einsum + zero/copy buffer"))
    cgs = O.linear_grad_sample(ca, cb)[0] if with_cpu else None
    yield row("sumsq_rows", "a10", "C2 n=128 P=16.8M f32", timed(lambda: K.sumsq_rows([gs])), "hbm", gs.numel() * 4,
              cpu(lambda: cgs.reshape(8, -1).norm(2, dim=-1), 16, "8 of 128 samples"))
    _, clip = K.clip_factor(ss.reshape(1, -1), 1.0)
    out = torch.empty(d, d, device=dev)
    yield row("clip_accumulate", "a10", "C2 n=128 P=16.8M f32", timed(lambda: K.clip_accumulate([gs], clip, [out], False)),
              "hbm", gs.numel() * 4 + out.numel() * 4,
              cpu(lambda: O.clip_and_accumulate([cgs], 1.0), 16, "8 of 128 samples, norm + clip + einsum"))
    gs16 = gs.bfloat16()  # the same tensor as a bf16 model's hooks would hold it
    out16 = torch.empty(d, d, device=dev, dtype=torch.bfloat16)
    yield row("clip_accumulate", "a10", "C2 shape in bf16: n=128 P=16.8M", timed(lambda: K.clip_accumulate([gs16], clip, [out16], False)),
              "hbm", gs16.numel() * 2 + out16.numel() * 2)
    yield row("sumsq_rows", "a10", "C2 shape in bf16: n=128 P=16.8M", timed(lambda: K.sumsq_rows([gs16])), "hbm", gs16.numel() * 2)
    del gs16, out16
    g = torch.empty_like(out)
    csum = torch.zeros(d, d) if with_cpu else None
    yield row("add_noise", "a11", "C2 P=16.8M f32", timed(lambda: K.add_noise(out, g, 1.0, 128.0, 1, 0)), "hbm", 2 * out.numel() * 4,
              cpu(lambda: O.add_noise_and_scale([csum], [csum.shape], 1.0, 1.0, 128), 1, "full size"))
    yield row("linear_bias_gs", "a1", "C2 n=128 out=4096 f32", timed(lambda: K.linear_bias_grad_sample(b)), "hbm", 2 * n * d * 4)
    del gs, out, g, cgs, csum
    # ---- Linear per-sample gradients with a sequence dimension (fp32 MFMA)
    n, T, i, o = 16, 256, 1024, 1024
    a, b = torch.randn(n, T, i, device=dev), torch.randn(n, T, o, device=dev)
    ca, cb = a[:4].cpu(), b[:4].cpu()
    yield row("linear_gs (T>1, fp32 MFMA)", "a1", "n=16 T=256 1024x1024 f32", timed(lambda: K.linear_grad_sample(b, a)),
              "mfma_fp32", 2.0 * n * T * i * o, cpu(lambda: O.linear_grad_sample(ca, cb), 4, "4 of 16 samples"))
    a3, b3 = torch.randn(16, 1024, 2048, device=dev), torch.randn(16, 1024, 1024, device=dev)
    yield row("linear_gs (T>1, fp32 MFMA)", "a1", "n=16 T=1024 2048->1024 f32", timed(lambda: K.linear_grad_sample(b3, a3)),
              "mfma_fp32", 2.0 * 16 * 1024 * 2048 * 1024)
    del a3, b3
    a16, b16 = a.bfloat16(), b.bfloat16()
    yield row("linear_gs (T>1, bf16 MFMA)", "a1", "n=16 T=256 1024x1024 bf16",
              timed(lambda: K.linear_grad_sample(b16, a16)), "mfma_bf16", 2.0 * n * T * i * o)
    n2, T2 = 16, 1024
    a2 = torch.randn(n2, T2, 2048, device=dev).bfloat16()
    for o2 in (1024, 5632):
        b2 = torch.randn(n2, T2, o2, device=dev).bfloat16()
        yield row("linear_gs (T>1, bf16 MFMA)", "a1", f"n=16 T=1024 2048->{o2} bf16",
                  timed(lambda: K.linear_grad_sample(b2, a2)), "mfma_bf16", 2.0 * n2 * T2 * 2048 * o2)
    del a16, b16, a2, b2
    # ---- C3 / C5: ghost norms, bf16
    for cfg, n, T, layers in (
        ("C3", 32, 512, [(1024, 4096, "fc1"), (4096, 1024, "fc2")]),
        ("C5", 16, 1024, [(2048, 2048, "q/o"), (2048, 512, "k/v"), (2048, 5632, "gate/up"), (5632, 2048, "down"),
                          (2048, 32000, "lm_head")]),
    ):
        tri, full = tri_tiles(T)
        for i, o, name in layers:
            a = torch.randn(n, T, i, device=dev).bfloat16()
            b = (torch.randn(n, T, o, device=dev) * 0.02).bfloat16()
            ms = timed(lambda: K.linear_ghost_norm(b, a, want_weight=True, want_bias=False))
            ca, cb = a[:1].cpu(), b[:1].cpu()
            gram, direct = T * T * (i + o) * tri / full, float(T) * i * o
            thin = direct < 0.9 * gram  # the library's rule: form the gradient tiles and square them
            yield row("linear_ghost_norm", "a2", f"{cfg} {name} n={n} T={T} {i}->{o} bf16" + (" (direct)" if thin else ""),
                      ms, "mfma_bf16", 2.0 * n * (direct if thin else gram),
                      cpu(lambda: O.linear_norm_sample(ca, cb), n, f"1 of {n} samples, bf16 bmm Grams"))
            del a, b
    # ... and pooled: all Linear layers of a backward pass in one launch (what a ghost-clipping step runs)
    for cfg, n, T, layers in (
        ("C3 fc1 + fc2", 32, 512, [(1024, 4096), (4096, 1024)]),
        ("C5 all 29 Linear layers (k/v by the direct route)", 16, 1024,
         [(2048, 2048), (2048, 512), (2048, 512), (2048, 2048), (2048, 5632), (2048, 5632), (5632, 2048)] * 4 + [(2048, 32000)]),
    ):
        tri, full = tri_tiles(T)
        items, work = [], 0.0
        for i, o in layers:
            a = torch.randn(n, T, i, device=dev).bfloat16()
            b = (torch.randn(n, T, o, device=dev) * 0.02).bfloat16()
            items.append((b, a, 1.0, torch.empty(n, device=dev), None))
            gram, direct = T * T * (i + o) * tri / full, float(T) * i * o
            work += 2.0 * n * (direct if direct < 0.9 * gram else gram)
        yield row("linear_ghost_norm_multi", "a2", f"{cfg} pooled, n={n} T={T} bf16",
                  timed(lambda: K.linear_ghost_norm_multi(items)), "mfma_bf16", work)
        del items
    # the clip-weighted sum of the same layers from the same operands (what replaces the second backward pass)
    for cfg, n, T, layers in (
        ("C3", 32, 512, [(1024, 4096, "fc1")]),
        ("C5", 16, 1024, [(2048, 2048, "q/o"), (2048, 512, "k/v"), (2048, 5632, "gate/up"), (2048, 32000, "lm_head")]),
    ):
        for i, o, name in layers:
            a = torch.randn(n, T, i, device=dev).bfloat16()
            b = (torch.randn(n, T, o, device=dev) * 0.02).bfloat16()
            c = torch.rand(n, device=dev) * 0.9 + 0.1
            ca, cb, cc = a[:1].cpu().float(), b[:1].cpu().float(), c[:1].cpu()
            yield row("linear_weighted_sum", "a9", f"{cfg} {name} n={n} T={T} {i}->{o} bf16",
                      timed(lambda: K.linear_weighted_sum(b, a, c)), "mfma_bf16", 2.0 * n * T * i * o,
                      cpu(lambda: torch.einsum("n,nij->ij", cc, O.linear_grad_sample(ca, cb)[0]), n,
                          f"1 of {n} samples, fp32 einsum + weighted sum"))
            del a, b
    # ... and pooled: the clipped sums of all of C5's Linear layers in one launch
    n, T = 16, 1024
    layers = [(2048, 2048), (2048, 512), (2048, 512), (2048, 2048), (2048, 5632), (2048, 5632), (5632, 2048)] * 4 + [(2048, 32000)]
    c = torch.rand(n, device=dev) * 0.9 + 0.1
    items = [((torch.randn(n, T, o, device=dev) * 0.02).bfloat16(), torch.randn(n, T, i, device=dev).bfloat16(), c, 1.0)
             for i, o in layers]
    yield row("linear_weighted_sum_multi", "a9", "C5 all 29 Linear layers pooled, n=16 T=1024 bf16",
              timed(lambda: K.linear_weighted_sum_multi(items)), "mfma_bf16", sum(2.0 * n * T * i * o for i, o in layers))
    del items
    # ... and C3's two layers pooled: too few tiles for the GPU, so the samples are cut into pieces inside the call
    n, T = 32, 512
    c = torch.rand(n, device=dev) * 0.9 + 0.1
    items = [((torch.randn(n, T, o, device=dev) * 0.02).bfloat16(), torch.randn(n, T, i, device=dev).bfloat16(), c, 1.0)
             for i, o in ((1024, 4096), (4096, 1024))]
    cpu_items = [(bb[:1].cpu().float(), aa[:1].cpu().float()) for bb, aa, _, _ in items]
    cc = c[:1].cpu()
    yield row("linear_weighted_sum_multi", "a9", "C3 fc1 + fc2 pooled (two pieces), n=32 T=512 bf16",
              timed(lambda: K.linear_weighted_sum_multi(items)), "mfma_bf16", 2 * 2.0 * n * T * 1024 * 4096,
              cpu(lambda: [torch.einsum("n,nij->ij", cc, O.linear_grad_sample(aa, bb)[0]) for bb, aa in cpu_items], n,
                  f"1 of {n} samples, both layers, fp32 einsum + weighted sum"))
    yield row("linear_bias_weighted_sum", "a9", "C3 fc1 bias n=32 T=512 out=4096 bf16",
              timed(lambda: K.linear_bias_weighted_sum(items[0][0], c)), "hbm", n * T * 4096 * 2,
              cpu(lambda: torch.einsum("n,ni->i", cc, O.linear_grad_sample(cpu_items[0][1], cpu_items[0][0])[1]), n,
                  f"1 of {n} samples, fp32 sum over positions + weighted sum"))
    del items
    # fp32 operands: the direct-load fp32 kernel with the coefficients on its accumulators, and the weighted-row
    # kernel for a sequence length that is not a whole number of k tiles
    c = torch.rand(16, device=dev) * 0.9 + 0.1
    a, b = torch.randn(16, 256, 1024, device=dev), torch.randn(16, 256, 1024, device=dev)
    ca, cb, cc = a[:4].cpu(), b[:4].cpu(), c[:4].cpu()
    yield row("linear_weighted_sum (fp32)", "a9", "n=16 T=256 1024x1024 f32",
              timed(lambda: K.linear_weighted_sum(b, a, c)), "mfma_fp32", 2.0 * 16 * 256 * 1024 * 1024,
              cpu(lambda: torch.einsum("n,nij->ij", cc, O.linear_grad_sample(ca, cb)[0]), 4, "4 of 16 samples, einsum + weighted sum"))
    a, b = torch.randn(16, 250, 1024, device=dev), torch.randn(16, 250, 1024, device=dev)
    yield row("linear_weighted_sum (fp32, weighted rows)", "a9", "n=16 T=250 1024x1024 f32",
              timed(lambda: K.linear_weighted_sum(b, a, c)), "mfma_fp32", 2.0 * 16 * 250 * 1024 * 1024)
    del a, b
    # the same kernel on fp32 operands
    tri, full = tri_tiles(1024)
    a = torch.randn(16, 1024, 2048, device=dev)
    b = torch.randn(16, 1024, 2048, device=dev) * 0.02
    yield row("linear_ghost_norm", "a2", "C5 q/o shape in fp32: n=16 T=1024 2048->2048 f32",
              timed(lambda: K.linear_ghost_norm(b, a, want_weight=True, want_bias=False)), "mfma_fp32",
              2.0 * 16 * 1024 * 1024 * 4096 * tri / full)
    del a, b
    # a low-rank adapter on C5's width: the direct route
    a = torch.randn(16, 1024, 2048, device=dev).bfloat16()
    b = (torch.randn(16, 1024, 16, device=dev) * 0.02).bfloat16()
    ca, cb = a[:1].cpu(), b[:1].cpu()
    yield row("linear_ghost_norm", "a2", "rank-16 adapter n=16 T=1024 2048->16 bf16 (direct)",
              timed(lambda: K.linear_ghost_norm(b, a, want_weight=True, want_bias=False)), "mfma_bf16",
              2.0 * 16 * 1024 * 2048 * 16, cpu(lambda: O.linear_norm_sample(ca, cb), 16, "1 of 16 samples, bf16 bmm Grams"))
    del a, b
    # ---- C5: embedding ghost norm, RMSNorm, noise over all parameters (bf16)
    n, T, D, V = 16, 1024, 2048, 32000
    ids = torch.randint(0, V, (n, T), device=dev)
    b = (torch.randn(n, T, D, device=dev) * 0.02).bfloat16()
    x = torch.randn(n, T, D, device=dev).bfloat16()
    cids, cb, cx = ids[:4].cpu(), b[:4].cpu(), x[:4].cpu()
    yield row("embedding_ghost_norm", "a5", "C5 n=16 T=1024 D=2048 bf16", timed(lambda: K.embedding_ghost_norm(ids, b)),
              "hbm", b.numel() * 2 + ids.numel() * 8,
              cpu(lambda: O.embedding_norm_sample(cids, cb), 4, "4 of 16 samples"))
    cw = torch.rand(n, device=dev) * 0.9 + 0.1
    ccw = cw[:1].cpu()
    yield row("embedding_weighted_sum", "a9", "C5 n=16 T=1024 V=32000 D=2048 bf16",
              timed(lambda: K.embedding_weighted_sum(ids, b, cw, V)), "hbm", b.numel() * 2 + V * D * 2 + ids.numel() * 8,
              cpu(lambda: torch.einsum("n,nvd->vd", ccw, O.embedding_grad_sample(cids[:1], cb[:1].float(), V)), n,
                  f"1 of {n} samples, per-sample table + weighted sum"))
    yield row("rms_norm_gs", "a6", "C5 n=16 T=1024 D=2048 bf16", timed(lambda: K.rms_norm_grad_sample(x, b, D, 1e-5)),
              "hbm", 2 * b.numel() * 2, cpu(lambda: O.rms_norm_grad_sample(cx, cb, (D,), 1e-5), 4, "4 of 16 samples"))
    ah = torch.randn(n, T, D, device=dev).bfloat16()
    gh = (torch.randn(n, T, V, device=dev) * 0.01).bfloat16()
    yield row("tied_embedding_cross", "a5+a2", "C5 tied n=16 T=1024 D=2048 V=32000 bf16",
              timed(lambda: K.tied_embedding_cross_term(ids, b, ah, gh)), "mfma_bf16", 2.0 * n * T * T * D,
              cpu(lambda: O.tied_embedding_norm_sample(cids[:1], cb[:1].float(), ah[:1].cpu().float(), gh[:1].cpu().float()),
                  16, "1 of 16 samples, both gradients materialised"))
    del ah, gh
    small = 2
    idsm = torch.randint(0, V, (small, T), device=dev)
    cidm, cbm = idsm.cpu(), b[:small].cpu()
    yield row("embedding_gs", "a4", f"n={small} T=1024 V=32000 D=2048 bf16", timed(lambda: K.embedding_grad_sample(idsm, b[:small], V)),
              "hbm", small * V * D * 2 + small * T * D * 2,
              cpu(lambda: O.embedding_grad_sample(cidm, cbm, V), 1, "full size"))
    P = 245_900_000
    sm_, gr_ = torch.randn(P, device=dev).bfloat16(), torch.empty(P, device=dev, dtype=torch.bfloat16)
    csum = torch.zeros(P // 10, dtype=torch.bfloat16) if with_cpu else None
    yield row("add_noise", "a11", "C5 P=245.9M bf16", timed(lambda: K.add_noise(sm_, gr_, 0.8, 16.0, 1, 0)), "hbm", 2 * P * 2,
              cpu(lambda: O.add_noise_and_scale([csum], [csum.shape], 0.8, 1.0, 16), 10, "a tenth of the elements"))
    del sm_, gr_, x, b
    # ---- C4: conv 64->64 3x3 on 32x32, GroupNorm(32, 64), fp32, batch 256
    n = 256
    x, b = torch.randn(n, 64, 32, 32, device=dev), torch.randn(n, 64, 32, 32, device=dev)
    cx, cb = x[:16].cpu(), b[:16].cpu()
    yield row("conv2d_gs", "a3", "C4 n=256 64->64 3x3 32x32 f32",
              timed(lambda: K.conv2d_grad_sample(x, b, (3, 3), (1, 1), (1, 1, 1, 1), (1, 1), 1)), "mfma_fp32",
              2.0 * n * 64 * 576 * 1024,
              cpu(lambda: O.conv2d_grad_sample(cx, cb, kernel_size=(3, 3), padding=(1, 1), stride=(1, 1), dilation=(1, 1), groups=1),
                  16, "16 of 256 samples, unfold + einsum"))
    yield row("conv2d_gs (norm only)", "a3", "C4 n=256 64->64 3x3 32x32 f32, gradient not stored",
              timed(lambda: K.conv2d_grad_sample(x, b, (3, 3), (1, 1), (1, 1, 1, 1), (1, 1), 1, norm_only=True)), "mfma_fp32",
              2.0 * n * 64 * 576 * 1024)
    x16, b16 = x.bfloat16(), b.bfloat16()
    yield row("conv2d_gs (bf16 MFMA)", "a3", "C4 shape in bf16: n=256 64->64 3x3 32x32",
              timed(lambda: K.conv2d_grad_sample(x16, b16, (3, 3), (1, 1), (1, 1, 1, 1), (1, 1), 1)), "mfma_bf16",
              2.0 * n * 64 * 576 * 1024)
    x16, b16 = torch.randn(64, 128, 28, 28, device=dev).bfloat16(), torch.randn(64, 128, 28, 28, device=dev).bfloat16()
    yield row("conv2d_gs (bf16 MFMA)", "a3", "n=64 128->128 3x3 28x28 bf16",
              timed(lambda: K.conv2d_grad_sample(x16, b16, (3, 3), (1, 1), (1, 1, 1, 1), (1, 1), 1)), "mfma_bf16",
              2.0 * 64 * 128 * 1152 * 784)
    del x16, b16
    yield row("group_norm_gs", "a6", "C4 n=256 C=64 G=32 32x32 f32", timed(lambda: K.group_norm_grad_sample(x, b, 32, 1e-5)),
              "hbm", 2 * x.numel() * 4, cpu(lambda: O.group_norm_grad_sample(cx, cb, 32, 1e-5), 16, "16 of 256 samples"))
    yield row("conv_bias_gs", "a3", "C4 n=256 O=64 32x32 f32", timed(lambda: K.conv_bias_grad_sample(b)), "hbm", b.numel() * 4)
    # ---- C1: the small CNN's layers, fp32, batch 256
    n = 256
    x, b = torch.randn(n, 1, 28, 28, device=dev), torch.randn(n, 16, 14, 14, device=dev)
    yield row("conv2d_gs", "a3", "C1 conv1 n=256 1->16 k8 s2 p3 f32",
              timed(lambda: K.conv2d_grad_sample(x, b, (8, 8), (2, 2), (3, 3, 3, 3), (1, 1), 1)), "mfma_fp32",
              2.0 * n * 16 * 64 * 196)
    x, b = torch.randn(n, 16, 13, 13, device=dev), torch.randn(n, 32, 5, 5, device=dev)
    yield row("conv2d_gs", "a3", "C1 conv2 n=256 16->32 k4 s2 f32",
              timed(lambda: K.conv2d_grad_sample(x, b, (4, 4), (2, 2), (0, 0, 0, 0), (1, 1), 1)), "mfma_fp32",
              2.0 * n * 32 * 256 * 25)
    # ---- C1: the whole optimizer step of the small CNN as one launch (factors, clipped sum, noise, scaling)
    sizes = [1024, 16, 8192, 32, 16384, 32, 320, 10]
    gsl = [torch.randn(n, P, device=dev) for P in sizes]
    ssl = [g.pow(2).sum(1) for g in gsl]
    grl = [torch.empty(P, device=dev) for P in sizes]
    sml = [torch.empty(P, device=dev) for P in sizes]
    yield row("clip_noise_step", "a10+a11", "C1 n=256 P=26010 (8 tensors) f32",
              timed(lambda: K.clip_noise_step(gsl, ssl, grl, sml, 1.0, 1.1, 256.0, 1, 0)), "hbm", (n + 2) * sum(sizes) * 4)


def run_workload(name: str, dev, steps: int, warmup: int, all_timers: bool = False, calibrate_copy: bool = False,
                 with_plain: bool = False) -> dict:
    """``warmup`` untimed steps, then ``steps`` timed steps of one configuration between device
    synchronisations; HIP events on the launch stream around the roofline kernel's entry point."""
    from opacus_amd import kernels

    w = WORKLOADS[name](dev)
    step = w["step"]
    for _ in range(warmup):
        step()
    if calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev)  # 1 GiB read + 1 GiB written
        dst = torch.empty_like(src)
        dst.copy_(src)
        del src, dst
    torch.cuda.synchronize()
    # HIP events around the dominant kernel's entry point only, unless every entry point is asked for
    only = None if all_timers else {w["roofline"]["timer"]} | {r["timer"] for r in w.get("roofline_also", {}).values()}
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]  # step boundaries on the launch stream
    with kernels.record_kernel_times(only=only) as times:
        t0 = time.perf_counter()
        marks[0].record()
        for i in range(steps):
            step()
            marks[i + 1].record()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    per_step = sorted(a.elapsed_time(b) for a, b in zip(marks, marks[1:]))

    kernel_ms = {k: sum(s.elapsed_time(e) for s, e in v) / steps for k, v in times.items()}

    def roof(spec: dict) -> dict:
        r = dict(spec)
        spans = [s.elapsed_time(e) for s, e in times.get(r.pop("timer"), [])]
        if "work_per_step" in r:  # several launches per step share the work figure
            work, ms = r.pop("work_per_step"), sum(spans) / steps
            r["launches_per_step"] = len(spans) // steps
        else:
            work, ms = r.pop("work_per_launch"), sum(spans) / max(len(spans), 1)
        scale = 1e9 if r["unit"] == "GB/s" else 1e12
        achieved = work / (ms * 1e-3) / scale if ms > 0 else 0.0
        out = {
            "kernel": r["kernel"], "bound": r["bound"], "achieved": achieved, "peak": r["peak"], "unit": r["unit"],
            "frac": achieved / r["peak"], "traffic": r["traffic"], "algorithmic_work": work, "kernel_ms": ms,
        }
        for key in ("traffic_source", "launches_per_step"):
            if key in r:
                out[key] = r[key]
        return out

    roofline = roof(w["roofline"])
    extra = dict(w["extra"])
    plain = None
    if with_plain and "plain" in w:
        plain = time_plain_step(w, steps, warmup)
    for key, spec in w.get("roofline_also", {}).items():  # the configuration's other contraction kernel
        extra[key] = roof(spec)
    return {
        "workload": w["workload"], "dtype": w["dtype"], "global_batch": w["n"], "steps": steps, "warmup": warmup,
        "ms_per_step": elapsed / steps * 1e3, "samples_per_s": w["n"] * steps / elapsed,
        # the middle step's span on the device: a single stalled step moves the mean of a short run, not this
        "ms_per_step_median": per_step[len(per_step) // 2] if per_step else None,
        "kernel_ms_per_step": kernel_ms, "extra": extra, "roofline": roofline, "plain_step": plain,
    }


def time_plain_step(w: dict, steps: int, warmup: int) -> dict:
    """The same network, batch and loss without any wrapper: forward, backward, SGD (the switch
    --disable-dp of the reference's examples/vision_benchmark.py:65, 259), timed in this process by
    the loop that times the DP step: ``warmup`` untimed steps, ``steps`` timed ones between device
    synchronisations."""
    step = w["plain"]()
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(steps):
        step()
        marks[i + 1].record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    per_step = sorted(a.elapsed_time(b) for a, b in zip(marks, marks[1:]))
    return {"ms_per_step": elapsed / steps * 1e3, "ms_per_step_median": per_step[len(per_step) // 2],
            "samples_per_s": w["n"] * steps / elapsed, "steps": steps, "warmup": warmup,
            "what": "same model, batch and loss, no DP wrapper: forward + backward + SGD"}


# Steps of the other configurations inside the default run: enough for a stable mean, few
# enough that the whole run stays within minutes (a c5 step takes 43-65 ms, the others 1-2 ms).
OTHER_CONFIGS = {"c1": (20, 5), "c3": (20, 5), "c4": (20, 5), "c5": (10, 3)}


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default=None,
                    help="time this configuration alone (default: c2 as the headline, then c1, c3, c4, c5 under 'configs')")
    ap.add_argument("--headline-only", action="store_true", help="config 2 only, without the 'configs' object")
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU oracle timings")
    ap.add_argument("--no-plain-step", action="store_true",
                    help="skip timing the same model without DP (plain_step) beside each configuration")
    ap.add_argument("--all-kernel-timers", action="store_true",
                    help="HIP-event timers around every entry point of the library (kernel_ms_per_step lists them all); "
                         "by default only the roofline kernel's entry point is timed")
    ap.add_argument(
        "--calibrate-copy",
        action="store_true",
        help="also run one 1 GiB device-to-device copy before the timed region (a dispatch of known "
        "traffic against which profiler byte counters can be scaled)",
    )
    ap.add_argument(
        "--kernels",
        action="store_true",
        help="instead of a training step, time every kernel of the library on its own at the five "
        "configurations' shapes and print one JSON line per kernel",
    )
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build uses one GPU; run with --gpus 1 (a larger count is not measured)")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP kernels have no CPU path")

    dev = torch.device("cuda:0")
    if args.kernels:
        for r in kernel_table(dev, with_cpu=not args.no_cpu_baseline):
            print(json.dumps(r), flush=True)
        return
    head_name = args.workload or "c2"
    head = run_workload(head_name, dev, args.steps, args.warmup, args.all_kernel_timers, args.calibrate_copy,
                        with_plain=not args.no_plain_step)
    out = {
        "metric": "dp_sgd_step_samples_per_sec",
        "value": head["samples_per_s"],
        "unit": "samples/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": head["dtype"],
        "data": "synthetic",
        "config": {"workload": head["workload"], "global_batch": head["global_batch"],
                   "kernel_ms_per_step": head["kernel_ms_per_step"], "ms_per_step_median": head["ms_per_step_median"],
                   **head["extra"]},
        "roofline": head["roofline"],
    }
    if head["plain_step"]:
        out["plain_step"] = head["plain_step"]
        out["dp_over_plain"] = head["ms_per_step"] / head["plain_step"]["ms_per_step"]
    cpu_ok = not args.no_cpu_baseline and head_name.rstrip("stdp") in ("c1", "c2", "c3", "c4", "c5")
    if cpu_ok:
        out["cpu_baseline"] = cpu_baseline(head_name.rstrip("stdp"))
    if args.workload is None and not args.headline_only:
        configs = {}
        d = run_workload("c2l", dev, args.steps, args.warmup, args.all_kernel_timers)
        configs["c2"] = {"lazy": {"ms_per_step": d["ms_per_step"], "ms_per_step_median": d["ms_per_step_median"],
                                  "samples_per_s": d["samples_per_s"], "workload": d["workload"], "roofline": d["roofline"],
                                  "note": "opt-in mode, beside the materialising headline above, which is the step "
                                          "BASELINE's metric is quoted on"}}
        for name, (k, wu) in OTHER_CONFIGS.items():
            torch.cuda.empty_cache()
            k, wu = min(k, args.steps), min(wu, max(args.warmup, 1))
            r = run_workload(name, dev, k, wu, args.all_kernel_timers, with_plain=not args.no_plain_step)
            entry = {key: r[key] for key in ("workload", "dtype", "global_batch", "steps", "warmup", "ms_per_step",
                                             "ms_per_step_median", "samples_per_s", "roofline")}
            entry.update(r["extra"])
            if r["plain_step"]:
                entry["plain_step"] = r["plain_step"]
                entry["dp_over_plain"] = r["ms_per_step"] / r["plain_step"]["ms_per_step"]
            if name + "p" in WORKLOADS:  # the same configuration with the reference's two backward passes
                d = run_workload(name + "p", dev, k, wu, args.all_kernel_timers)
                entry["two_backward_passes"] = {"ms_per_step": d["ms_per_step"], "ms_per_step_median": d["ms_per_step_median"],
                    "samples_per_s": d["samples_per_s"],
                                                "single_backward": False}
            if name + "t" in WORKLOADS:  # the same decoder with embedding table and LM head sharing one parameter
                d = run_workload(name + "t", dev, k, wu, args.all_kernel_timers)
                entry["tied_embeddings"] = {"ms_per_step": d["ms_per_step"], "ms_per_step_median": d["ms_per_step_median"],
                    "samples_per_s": d["samples_per_s"],
                                            "workload": d["workload"]}
            if name + "d" in WORKLOADS:  # the same configuration with the library's default hooks
                d = run_workload(name + "d", dev, k, wu, args.all_kernel_timers)
                entry["default_hooks"] = {"ms_per_step": d["ms_per_step"], "ms_per_step_median": d["ms_per_step_median"],
                    "samples_per_s": d["samples_per_s"],
                                          "autograd_weight_grads": True}
            if not args.no_cpu_baseline:
                entry["cpu_baseline"] = cpu_baseline(name)
            configs[name] = entry
        out["configs"] = configs
    print(json.dumps(out))


if __name__ == "__main__":
    main()
