"""How the GPU tests compare a kernel's output with the oracle's.

One bar `rel` (fp32: 1e-5, bf16: 2e-2) is applied at three scales, and the worst of the three
is what a test asserts on:

  * tensor scale:   max |err|    <= rel * max |want|        over the whole tensor;
  * sample scale:   max |err_n|  <= rel * max |want_n|      for every sample n (first dimension),
                    so that a sample whose values are small next to the batch's largest is held
                    to its own size;
  * element scale:  |err|        <= rel * (|want| + rms(want_n))  for every element, so that an
                    error confined to small entries (a dropped contribution in a near-zero row, a
                    wrong tail element) shows, while an entry that is small by cancellation is
                    allowed the rounding of the terms that cancelled (rms of its sample).

The reference's own tests use atol=1e-5/rtol=1e-4 for per-sample gradients
(opacus/tests/grad_samples/common.py:50-51); these bars are tighter.
"""

import torch


def rel_measures(got: torch.Tensor, want: torch.Tensor):
    """(tensor-scale, sample-scale, element-scale) relative errors as floats."""
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    assert got.shape == want.shape, f"shape {tuple(got.shape)} != {tuple(want.shape)}"
    if want.numel() == 0:
        return 0.0, 0.0, 0.0
    err = (got - want).abs()
    tiny = 1e-300
    tensor = (err.max() / want.abs().max().clamp_min(tiny)).item()
    if want.dim() >= 2:
        e2, w2 = err.flatten(1), want.flatten(1)
        smax = w2.abs().max(dim=1).values
        emax = e2.max(dim=1).values
        sample = torch.where(emax == 0, torch.zeros_like(emax), emax / smax.clamp_min(tiny)).max().item()
        rms = w2.pow(2).mean(dim=1, keepdim=True).sqrt()
        denom = (w2.abs() + rms).clamp_min(tiny)
        element = torch.where(e2 == 0, torch.zeros_like(e2), e2 / denom).max().item()
    else:
        # a vector (per-sample norms, a bias-shaped sum): one group, every entry against its own
        # size plus the vector's rms
        sample = tensor
        rms = want.pow(2).mean().sqrt()
        element = torch.where(err == 0, torch.zeros_like(err), err / (want.abs() + rms).clamp_min(tiny)).max().item()
    return tensor, sample, element


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """The worst of the three measures."""
    return max(rel_measures(got, want))


def assert_rel(got: torch.Tensor, want: torch.Tensor, rel: float, what: str = "") -> None:
    assert tuple(got.shape) == tuple(want.shape), f"{what}: shape {tuple(got.shape)} != {tuple(want.shape)}"
    t, s, e = rel_measures(got, want)
    assert max(t, s, e) <= rel, f"{what}: relative error tensor-scale {t:.2e}, sample-scale {s:.2e}, element-scale {e:.2e} > {rel:.1e}"
