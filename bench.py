"""DP-SGD step throughput on one MI355X: ``python bench.py --gpus 1 --steps K --warmup W``.

Default workload (the one the headline metric is quoted on): a single
``nn.Linear(4096, 4096, bias=True)`` in fp32, batch 128, one position per sample, hooks
mode: forward, backward (per-sample gradients, 128 x 4096 x 4096 fp32 = 8.59 GB), then
``DPOptimizer.step`` (clip at C = 1, accumulate, noise sigma = 1, SGD update) and
``zero_grad``. Inputs are synthetic N(0,1) tensors resident in HBM before the clock starts.

Prints ONE JSON line. ``roofline`` describes the dominant kernel of the step (the
clip-weighted sum over the batch, which streams the per-sample gradients once), timed
with HIP events on the launch stream inside the timed region. ``cpu_baseline`` is the
CPU oracle (a restatement of the reference's einsum path, allocation pattern included)
timed on this box's host cores on a bounded sample of the same workload.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

import torch
import torch.nn as nn

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
N, D_IN, D_OUT = 128, 4096, 4096
SIGMA, CLIP, LR = 1.0, 1.0, 0.05


def gpu_step_factory(dev):
    from opacus_amd import GradSampleModule
    from opacus_amd.optimizers import DPOptimizer

    torch.manual_seed(0)
    lin = nn.Linear(D_IN, D_OUT, bias=True)
    x = torch.randn(N, D_IN)
    b = torch.randn(N, D_OUT)
    model = GradSampleModule(lin.to(dev), loss_reduction="sum")
    opt = DPOptimizer(
        torch.optim.SGD(model.parameters(), lr=LR),
        noise_multiplier=SIGMA,
        max_grad_norm=CLIP,
        expected_batch_size=N,
        loss_reduction="sum",
    )
    x, b = x.to(dev), b.to(dev)

    def step():
        opt.zero_grad(set_to_none=True)
        y = model(x)
        y.backward(b)  # backprops ~ N(0,1) injected at the layer output
        opt.step()

    return step, model


def cpu_baseline(n_sample: int = 16, steps: int = 3) -> dict:
    """The oracle's DP-SGD step for the same layer on the host cores, on ``n_sample`` of the
    128 samples (every pass over per-sample data is linear in the batch size)."""
    from oracle import dp_oracle as O

    torch.manual_seed(0)
    lin = nn.Linear(D_IN, D_OUT, bias=True)
    x = torch.randn(n_sample, D_IN)
    b = torch.randn(n_sample, D_OUT)
    sgd = torch.optim.SGD(lin.parameters(), lr=LR)

    def step():
        sgd.zero_grad(set_to_none=True)
        y = lin(x)
        y.backward(b)
        bp = O.scale_backprops(b, n_sample, "sum")
        gs_w, gs_b = O.linear_grad_sample(x, bp)
        gs = [O.store_grad_sample(gs_w, n_sample), O.store_grad_sample(gs_b, n_sample)]
        _, _, summed = O.clip_and_accumulate(gs, CLIP)
        grads = O.add_noise_and_scale(summed, [lin.weight.shape, lin.bias.shape], SIGMA, CLIP, n_sample, "sum")
        lin.weight.grad, lin.bias.grad = grads
        sgd.step()

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
        "sample": f"{steps} steps at batch {n_sample} of {N} (per-sample passes are linear in the batch); "
        f"{os.cpu_count()} logical CPUs visible",
    }


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU oracle timing")
    ap.add_argument(
        "--calibrate-copy",
        action="store_true",
        help="also run one 1 GiB device-to-device copy before the timed region (a dispatch of known "
        "traffic against which profiler byte counters can be scaled)",
    )
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build uses one GPU; run with --gpus 1 (a larger count is not measured)")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP kernels have no CPU path")

    from opacus_amd import kernels

    dev = torch.device("cuda:0")
    step, model = gpu_step_factory(dev)
    for _ in range(args.warmup):
        step()
    if args.calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev)  # 1 GiB read + 1 GiB written
        dst = torch.empty_like(src)
        dst.copy_(src)
        del src, dst
    torch.cuda.synchronize()
    with kernels.record_kernel_times() as times:
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0

    ms_per_step = elapsed / args.steps * 1e3
    value = N * args.steps / elapsed

    # dominant kernel: the clip-weighted sum. One launch covers weight and bias:
    # reads n * P * 4 bytes, writes P * 4 bytes, P = 4096 * 4096 + 4096.
    P = D_OUT * D_IN + D_OUT
    algo_bytes = N * P * 4 + P * 4
    ca = [s.elapsed_time(e) for s, e in times.get("clip_accumulate", [])]
    ca_ms = sum(ca) / max(len(ca), 1)
    achieved = algo_bytes / (ca_ms * 1e-3) / 1e9 if ca_ms > 0 else 0.0
    kernel_ms = {k: sum(s.elapsed_time(e) for s, e in v) / args.steps for k, v in times.items()}

    out = {
        "metric": "dp_sgd_step_samples_per_sec",
        "value": value,
        "unit": "samples/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "Linear(4096->4096, bias) fp32, batch 128, T=1, hooks per-sample grad + clip(C=1) + noise(sigma=1) + SGD",
            "global_batch": N,
            "per_sample_grad_bytes": N * P * 4,
            "kernel_ms_per_step": kernel_ms,
        },
        "roofline": {
            "kernel": "clip_accumulate_kernel<float,float,vec,RS=1>",
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE (KiB per
            # dispatch), each scaled by what the counter reads for a 1 GiB device copy
            # (FETCH_SIZE x 2.000, WRITE_SIZE x 1.000): 8,390,854 + 65,552 KiB.
            "traffic": 8456406 * 1024,
            "algorithmic_bytes_per_launch": algo_bytes,
            "avg_launch_ms": ca_ms,
        },
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
