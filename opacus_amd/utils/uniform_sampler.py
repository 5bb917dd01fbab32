"""Poisson batch sampler (mirror of opacus/utils/uniform_sampler.py, single process)."""

from __future__ import annotations

from typing import Iterator, List, Optional

import torch
from torch.utils.data import Sampler


class UniformWithReplacementSampler(Sampler[List[int]]):
    """Every step, each of ``num_samples`` indices joins the batch independently with
    probability ``sample_rate``; ``steps`` batches per epoch, ``int(1 / sample_rate)`` by
    default (uniform_sampler.py:22-70). Batches vary in size and may be empty."""

    def __init__(self, *, num_samples: int, sample_rate: float, generator=None, steps: Optional[int] = None):
        if num_samples <= 0:
            raise ValueError(f"num_samples should be a positive integer value, but got num_samples={num_samples}")
        self.num_samples = num_samples
        self.sample_rate = sample_rate
        self.generator = generator
        self.steps = steps if steps is not None else int(1 / sample_rate)

    def __len__(self) -> int:
        return self.steps

    def __iter__(self) -> Iterator[List[int]]:
        for _ in range(self.steps):
            chosen = torch.rand(self.num_samples, generator=self.generator) < self.sample_rate
            yield chosen.nonzero(as_tuple=False).reshape(-1).tolist()
