"""DP optimizers on the HIP kernels; same names as ``opacus.optimizers``."""

from .adaclipoptimizer import AdaClipDPOptimizer
from .optimizer import DPOptimizer
from .optimizer_fast_gradient_clipping import DPOptimizerFastGradientClipping
from .perlayeroptimizer import DPPerLayerOptimizer

__all__ = [
    "AdaClipDPOptimizer",
    "DPOptimizer",
    "DPOptimizerFastGradientClipping",
    "DPPerLayerOptimizer",
    "get_optimizer_class",
]


def get_optimizer_class(clipping: str, distributed: bool, grad_sample_mode: str = None):
    """Optimizer class for a clipping strategy (opacus/optimizers/__init__.py:39-71).

    Built here: flat, per-layer and adaptive clipping on one GPU (ghost clipping with flat
    clipping only, as in the reference). Every distributed optimizer is outside this build.
    """
    if distributed:
        raise NotImplementedError("distributed DP optimizers are outside this build (one GPU)")
    if clipping == "flat":
        if grad_sample_mode == "ghost":
            return DPOptimizerFastGradientClipping
        if grad_sample_mode in (None, "hooks", "functorch"):
            return DPOptimizer
        raise NotImplementedError(f"grad_sample_mode={grad_sample_mode!r} is outside this build")
    if clipping == "per_layer" and grad_sample_mode in (None, "hooks", "functorch"):
        return DPPerLayerOptimizer
    if clipping == "adaptive" and grad_sample_mode in (None, "hooks", "functorch"):
        return AdaClipDPOptimizer
    raise ValueError(f"Unexpected optimizer parameters. Clipping: {clipping}, distributed: {distributed}")
