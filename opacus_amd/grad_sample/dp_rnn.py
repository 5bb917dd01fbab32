"""Samplers of ``RNNLinear``, the building block of DPRNN / DPGRU / DPLSTM
(mirror of opacus/grad_sample/dp_rnn.py).

The arithmetic is nn.Linear's. The hooks hand over all uses of the layer in one backward
pass stacked as ``[n, uses, features]``, so the sum over time steps happens inside the
contraction; for the same reason the ghost norm of the summed gradient is the Gram form over
the uses, which the reference does not have for this layer (it materialises the gradient).
"""

from __future__ import annotations

from ..layers.dp_rnn import RNNLinear
from .linear import compute_linear_grad_sample, compute_linear_norm_sample
from .utils import register_grad_sampler, register_norm_sampler

compute_rnn_linear_grad_sample = register_grad_sampler(RNNLinear)(compute_linear_grad_sample)
compute_rnn_linear_norm_sample = register_norm_sampler(RNNLinear)(compute_linear_norm_sample)
