"""Large logical batches from small physical ones (mirror of opacus/utils/batch_memory_manager.py).

A logical batch drawn by the data loader's batch sampler is cut into physical batches of at
most ``max_batch_size`` samples. Before each physical batch the optimizer is told whether a
real step follows it: for all pieces but the last, ``DPOptimizer.step`` only clips the
per-sample gradients and adds them into ``p.summed_grad`` (the accumulate form of the
clip-accumulate kernel) and ``zero_grad`` keeps that sum; the last piece adds noise, rescales
by the logical batch size and steps (optimizer.py:294-329, 506-572).
"""

from __future__ import annotations

import math
from typing import Iterator, List

from torch.utils.data import BatchSampler, DataLoader, Sampler


def _split(indices: List[int], max_batch_size: int) -> List[List[int]]:
    """``len(indices)`` cut into ``ceil(len / max)`` nearly equal consecutive pieces, the longer
    ones first: the split of ``numpy.array_split`` that the reference uses
    (batch_memory_manager.py:64-67)."""
    pieces = math.ceil(len(indices) / max_batch_size)
    base, extra = divmod(len(indices), pieces)
    out, lo = [], 0
    for k in range(pieces):
        hi = lo + base + (1 if k < extra else 0)
        out.append(list(indices[lo:hi]))
        lo = hi
    return out


class BatchSplittingSampler(Sampler[List[int]]):
    """Yields the wrapped batch sampler's index lists in pieces of at most ``max_batch_size``
    and queues, for every piece, whether the optimizer must skip the real step after it
    (batch_memory_manager.py:27-88). An empty logical batch passes through as one empty piece
    with a real step."""

    def __init__(self, *, sampler: Sampler[List[int]], max_batch_size: int, optimizer):
        if max_batch_size < 1:
            raise ValueError(f"max_batch_size must be positive, got {max_batch_size}")
        self.sampler = sampler
        self.max_batch_size = max_batch_size
        self.optimizer = optimizer

    def __iter__(self) -> Iterator[List[int]]:
        for logical in self.sampler:
            logical = list(logical)
            if not logical:
                self.optimizer.signal_skip_step(do_skip=False)
                yield []
                continue
            pieces = _split(logical, self.max_batch_size)
            for piece in pieces[:-1]:
                self.optimizer.signal_skip_step(do_skip=True)
                yield piece
            self.optimizer.signal_skip_step(do_skip=False)
            yield pieces[-1]

    def __len__(self) -> int:
        # an estimate, as in the reference: logical batches times pieces per logical batch
        if isinstance(self.sampler, BatchSampler):
            return math.ceil(len(self.sampler) * (self.sampler.batch_size / self.max_batch_size))
        rate, count = getattr(self.sampler, "sample_rate", None), getattr(self.sampler, "num_samples", None)
        if rate is not None and count is not None:  # Poisson-style samplers: expected batch size
            return math.ceil(len(self.sampler) * (rate * count / self.max_batch_size))
        return len(self.sampler)


def wrap_data_loader(*, data_loader: DataLoader, max_batch_size: int, optimizer) -> DataLoader:
    """A new ``DataLoader`` over the same dataset whose batch sampler is the given one wrapped
    in :class:`BatchSplittingSampler` (batch_memory_manager.py:91-124). The input loader is
    left as it is."""
    return DataLoader(
        dataset=data_loader.dataset,
        batch_sampler=BatchSplittingSampler(
            sampler=data_loader.batch_sampler, max_batch_size=max_batch_size, optimizer=optimizer
        ),
        num_workers=data_loader.num_workers,
        collate_fn=data_loader.collate_fn,
        pin_memory=data_loader.pin_memory,
        timeout=data_loader.timeout,
        worker_init_fn=data_loader.worker_init_fn,
        multiprocessing_context=data_loader.multiprocessing_context,
        generator=data_loader.generator,
        prefetch_factor=data_loader.prefetch_factor,
        persistent_workers=data_loader.persistent_workers,
    )


class BatchMemoryManager:
    """``with BatchMemoryManager(data_loader=dl, max_physical_batch_size=m, optimizer=opt) as dl2:``
    iterate ``dl2`` and call ``opt.step()`` / ``opt.zero_grad()`` after every physical batch as
    usual; only the last piece of a logical batch updates the model
    (batch_memory_manager.py:127-180)."""

    def __init__(self, *, data_loader: DataLoader, max_physical_batch_size: int, optimizer):
        self.data_loader = data_loader
        self.optimizer = optimizer
        self.max_physical_batch_size = max_physical_batch_size

    def __enter__(self) -> DataLoader:
        return wrap_data_loader(
            data_loader=self.data_loader, max_batch_size=self.max_physical_batch_size, optimizer=self.optimizer
        )

    def __exit__(self, exc_type, exc, tb):
        return None
