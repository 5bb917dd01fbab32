"""``params(optimizer)``: the trainable parameters an optimizer steps (opacus/optimizers/utils.py:21-33)."""

from __future__ import annotations

from typing import List

import torch.nn as nn
from torch.optim import Optimizer


def params(optimizer: Optimizer) -> List[nn.Parameter]:
    """Parameters of all groups that require grad, in group order."""
    return [p for group in optimizer.param_groups for p in group["params"] if p.requires_grad]
