"""DP optimizers on the HIP kernels; same names as ``opacus.optimizers``."""

from .optimizer import DPOptimizer
from .optimizer_fast_gradient_clipping import DPOptimizerFastGradientClipping

__all__ = ["DPOptimizer", "DPOptimizerFastGradientClipping", "get_optimizer_class"]


def get_optimizer_class(clipping: str, distributed: bool, grad_sample_mode: str = None):
    """Optimizer class for a clipping strategy (opacus/optimizers/__init__.py:39-71).

    Built here: flat clipping on one GPU, for the hooks and ghost modes. Per-layer and
    adaptive clipping and every distributed optimizer are outside this build.
    """
    if distributed:
        raise NotImplementedError("distributed DP optimizers are outside this build (one GPU)")
    if clipping == "flat":
        if grad_sample_mode == "ghost":
            return DPOptimizerFastGradientClipping
        if grad_sample_mode in (None, "hooks", "functorch"):
            return DPOptimizer
        raise NotImplementedError(f"grad_sample_mode={grad_sample_mode!r} is outside this build")
    if clipping in ("per_layer", "adaptive"):
        raise NotImplementedError(f"clipping={clipping!r} is outside this build: only flat clipping is implemented")
    raise ValueError(f"Unexpected optimizer parameters. Clipping: {clipping}, distributed: {distributed}")
