"""Per-sample gradients and per-sample gradient norms on hand-written HIP kernels.

Same names as ``opacus.grad_sample``; importing this package registers the samplers.
"""

from .grad_sample_module import GradSampleHooks, GradSampleModule, create_or_accumulate_grad_sample
from .grad_sample_module_fast_gradient_clipping import (
    GradSampleHooksFastGradientClipping,
    GradSampleModuleFastGradientClipping,
)
from .gsm_base import AbstractGradSampleHooks, AbstractGradSampleModule
from .lazy import LazyLinearGradSample
from .utils import (
    get_gsm_class,
    get_hooks_class,
    prepare_module,
    register_grad_sampler,
    register_norm_sampler,
    wrap_model,
)
from .conv import compute_conv_grad_sample  # noqa: E402
from .dp_multihead_attention import compute_sequence_bias_grad_sample  # noqa: E402
from .dp_rnn import compute_rnn_linear_grad_sample, compute_rnn_linear_norm_sample  # noqa: E402
from .embedding import (  # noqa: E402
    compute_embedding_grad_sample,
    compute_embedding_norm_sample,
    compute_embeddingbag_gradsampler,
)
from .group_norm import compute_group_norm_grad_sample  # noqa: E402
from .instance_norm import compute_instance_norm_grad_sample  # noqa: E402
from .layer_norm import compute_layer_norm_grad_sample  # noqa: E402
from .linear import compute_linear_grad_sample, compute_linear_norm_sample  # noqa: E402
from .rms_norm import compute_rms_norm_grad_sample  # noqa: E402

__all__ = [
    "GradSampleModule",
    "GradSampleHooks",
    "GradSampleModuleFastGradientClipping",
    "GradSampleHooksFastGradientClipping",
    "AbstractGradSampleModule",
    "AbstractGradSampleHooks",
    "LazyLinearGradSample",
    "register_grad_sampler",
    "register_norm_sampler",
    "create_or_accumulate_grad_sample",
    "prepare_module",
    "wrap_model",
    "get_gsm_class",
    "get_hooks_class",
]
