"""A per-sample gradient of an ``nn.Linear`` weight that is formed only when somebody reads it.

The per-sample gradient of a Linear weight is ``scale * b[n]^T a[n]`` (linear.py:41-48): ``n``
products of a ``[T, out]`` and a ``[T, in]`` matrix, stored as ``[n, out, in]``. What a DP-SGD
step needs from it is its norm per sample and its clip-weighted sum over the samples
(optimizers/optimizer.py:444-475), and both follow from the two factors without the
``[n, out, in]`` tensor: the norm from the rank-one closed form or the Gram contraction
(linear.py:54-93), the weighted sum from one contraction over samples and positions with the
clip factors as coefficients. With ``GradSampleModule(..., lazy_linear_grad_sample=True)``
``weight.grad_sample`` of such a layer is a :class:`LazyLinearGradSample`, which keeps the
factors; :class:`~opacus_amd.optimizers.DPOptimizer` reads norms and weighted sum from it, and
any other reader (a torch function, a method, an index) gets the tensor the eager sampler
would have stored, formed at that moment by the same kernel and kept from then on.
"""

from __future__ import annotations

from typing import Dict, List, Optional

import torch
import torch.nn as nn

from .. import kernels
from ._common import tag_sumsq


class LazyLinearGradSample:
    """Stands in for the ``[n, out, in]`` per-sample gradient of an ``nn.Linear`` weight.

    ``backprops`` is ``[n, *, out]``, ``activations`` ``[n, *, in]`` (batch first, as the hooks
    hand them to a sampler), ``scale`` what the sampler would have applied to the backprops.
    Not a ``torch.Tensor``: ``isinstance`` checks see that, everything else is forwarded to the
    materialised tensor.
    """

    def __init__(self, backprops: torch.Tensor, activations: torch.Tensor, scale: float = 1.0):
        self._b = backprops
        self._a = activations
        self._scale = float(scale)
        self._gs: Optional[torch.Tensor] = None
        self._sumsq: Optional[torch.Tensor] = None
        self._shape = torch.Size((backprops.shape[0], backprops.shape[-1], activations.shape[-1]))

    # ---- what can be said without the tensor ---------------------------------------------
    @property
    def shape(self) -> torch.Size:
        return self._shape

    @property
    def dtype(self) -> torch.dtype:
        return self._b.dtype

    @property
    def device(self) -> torch.device:
        return self._b.device

    @property
    def ndim(self) -> int:
        return 3

    @property
    def is_cuda(self) -> bool:
        return self._b.is_cuda

    @property
    def is_materialized(self) -> bool:
        return self._gs is not None

    def dim(self) -> int:
        return 3

    def size(self, d: Optional[int] = None):
        return self._shape if d is None else self._shape[d]

    def numel(self) -> int:
        return self._shape.numel()

    def __len__(self) -> int:
        return self._shape[0]

    def __repr__(self) -> str:
        state = "materialized" if self.is_materialized else "factors only"
        return f"LazyLinearGradSample(shape={tuple(self._shape)}, dtype={self.dtype}, device={self.device}, {state})"

    # ---- what the optimizer reads ----------------------------------------------------------
    @property
    def sumsq(self) -> torch.Tensor:
        """``float32[n]`` squared Frobenius norms of the per-sample gradients (linear.py:54-93)."""
        if self._gs is not None:
            # somebody may have written to the tensor since: its own cached squares know
            from ._common import cached_sumsq

            ss = cached_sumsq(self._gs)
            return ss if ss is not None else kernels.sumsq_rows([self._gs.reshape(len(self), -1)])[0]
        if self._sumsq is None:
            if len(self) == 0:
                self._sumsq = torch.zeros(0, dtype=torch.float32, device=self.device)
            else:
                norm, _ = kernels.linear_ghost_norm(self._b, self._a, scale=self._scale, want_weight=True, want_bias=False)
                self._sumsq = norm * norm
        return self._sumsq

    def weighted_sum(self, coef: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        """``sum_n coef[n] * grad_sample[n]`` as ``[out, in]`` (optimizer.py:457-466 for this
        parameter): from the factors while the tensor does not exist, from the tensor once it does
        (a reader may have changed it)."""
        out_dtype = out_dtype or self.dtype
        if self._gs is not None:
            out = torch.empty(self._shape[1:], dtype=out_dtype, device=self.device)
            kernels.clip_accumulate([self._gs], coef, [out], accumulate=False)
            return out
        return kernels.linear_weighted_sum(self._b, self._a, coef, scale=self._scale, out_dtype=out_dtype)

    # ---- everything else: the tensor itself --------------------------------------------------
    def materialize(self) -> torch.Tensor:
        """The ``[n, out, in]`` tensor, formed on the first call by the kernel the eager sampler
        uses (with its sums of squares attached) and kept; the factors are dropped."""
        if self._gs is None:
            gs, sumsq = kernels.linear_grad_sample(self._b, self._a, scale=self._scale)
            self._gs = tag_sumsq(gs, sumsq)
            self._b = self._b.new_empty((self._shape[0], 0, self._shape[1]))
            self._a = self._a.new_empty((self._shape[0], 0, self._shape[2]))
            self._sumsq = None
        return self._gs

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        def real(x):
            if isinstance(x, LazyLinearGradSample):
                return x.materialize()
            if isinstance(x, (list, tuple)):
                return type(x)(real(v) for v in x)
            return x

        return func(*real(args), **{k: real(v) for k, v in (kwargs or {}).items()})

    def __getattr__(self, name):
        # only reached for names this class does not define: methods and attributes of the tensor
        if name.startswith("__") and name.endswith("__"):
            raise AttributeError(name)
        return getattr(self.materialize(), name)

    def __getitem__(self, idx):
        return self.materialize()[idx]

    def __setitem__(self, idx, value):
        self.materialize()[idx] = value

    def __iter__(self):
        return iter(self.materialize())


def lazy_linear_grad_sample(
    layer: nn.Linear, activations: List[torch.Tensor], backprops: torch.Tensor, scale: float = 1.0
) -> Dict[nn.Parameter, object]:
    """What the Linear sampler returns (linear.py:29-51) with the weight's entry left as its two
    factors; the bias's ``[n, out]`` is small and formed at once."""
    ret: Dict[nn.Parameter, object] = {}
    if layer.weight.requires_grad:
        ret[layer.weight] = LazyLinearGradSample(backprops, activations[0], scale)
    if layer.bias is not None and layer.bias.requires_grad:
        ret[layer.bias] = kernels.linear_bias_grad_sample(backprops, scale=scale)
    return ret


def _forward_binary(name: str):
    def op(self, other):
        other = other.materialize() if isinstance(other, LazyLinearGradSample) else other
        return getattr(self.materialize(), name)(other)

    op.__name__ = name
    return op


for _name in (
    "__add__", "__radd__", "__iadd__", "__sub__", "__rsub__", "__isub__", "__mul__", "__rmul__", "__imul__",
    "__truediv__", "__rtruediv__", "__itruediv__", "__matmul__", "__rmatmul__", "__pow__", "__eq__", "__ne__",
    "__lt__", "__le__", "__gt__", "__ge__",
):
    setattr(LazyLinearGradSample, _name, _forward_binary(_name))
LazyLinearGradSample.__neg__ = lambda self: -self.materialize()
LazyLinearGradSample.__abs__ = lambda self: abs(self.materialize())
LazyLinearGradSample.__hash__ = object.__hash__
