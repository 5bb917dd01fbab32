"""MI355X-native DP-SGD hot path with the public surface of Opacus.

``GradSampleModule``, ``GradSampleModuleFastGradientClipping``, ``register_grad_sampler``,
``DPOptimizer`` and ``PrivacyEngine.make_private`` keep the reference's names, arguments
and error behaviour; the arithmetic runs in hand-written HIP kernels (``libdpsgd_hip.so``,
C ABI in ``include/dpk.h``) on the GPU that holds the tensors. There is no CPU path.
"""

from . import grad_sample, layers, optimizers
from .grad_sample import (
    GradSampleHooks,
    GradSampleHooksFastGradientClipping,
    GradSampleModule,
    GradSampleModuleFastGradientClipping,
    register_grad_sampler,
    register_norm_sampler,
)
from .optimizers import DPOptimizer, DPOptimizerFastGradientClipping
from .privacy_engine import PrivacyEngine
from .utils.fast_gradient_clipping_utils import DPLossFastGradientClipping, DPTensorFastGradientClipping

__version__ = "0.1.0"

__all__ = [
    "PrivacyEngine",
    "GradSampleModule",
    "GradSampleHooks",
    "GradSampleModuleFastGradientClipping",
    "GradSampleHooksFastGradientClipping",
    "DPOptimizer",
    "DPOptimizerFastGradientClipping",
    "DPLossFastGradientClipping",
    "DPTensorFastGradientClipping",
    "register_grad_sampler",
    "register_norm_sampler",
    "grad_sample",
    "layers",
    "optimizers",
]
