"""Synthetic token batches of the reference's benchmark, generated on the device.

Mirrors ``generate_batches_of_sequential_tokens`` (reference src/olmax/data/utils.py:36-66) and
the benchmark's ``DataLoader`` state protocol (src/integration_tests/train_transformer.py:50-99).
The reference draws the per-sequence start offsets with ``jax.random.randint`` from keys folded
with the batch and micro-batch index; the JAX bit-stream cannot be reproduced without JAX, so the
offsets come from a ``torch.Generator`` seeded with (seed, epoch, batch, micro-batch) instead --
same distribution (uniform on [0, V-1)), same integer arithmetic afterwards.
"""
from __future__ import annotations

from typing import Iterator, List, Tuple

import torch

from ._lib import check, i32, load, ptr, stream_ptr


def start_offsets(seed: int, epoch: int, batch_idx: int, microbatch_idx: int, num_instances: int,
                  vocab_size: int) -> torch.Tensor:
    """[num_instances] int32 offsets, uniform on [0, vocab_size - 1) (upper bound exclusive, as
    random.randint(key, shape, 0, vocab_size - 1) in the reference, data/utils.py:21)."""
    g = torch.Generator()
    g.manual_seed(((seed * 1000003 + epoch) * 1000003 + batch_idx) * 1000003 + microbatch_idx)
    return torch.randint(0, max(1, vocab_size - 1), (num_instances,), generator=g, dtype=torch.int32)


def sequential_tokens(offsets: torch.Tensor, sequence_length: int, vocab_size: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """(inputs, targets), both [B, S] int32 on the device of `offsets` (must be a GPU tensor)."""
    if not offsets.is_cuda:
        raise ValueError("sequential_tokens: offsets must live on the GPU (there is no CPU path)")
    offsets = offsets.to(torch.int32).contiguous()
    B = offsets.numel()
    inputs = torch.empty(B, sequence_length, device=offsets.device, dtype=torch.int32)
    targets = torch.empty_like(inputs)
    check(load().olmax_sequential_tokens(stream_ptr(), ptr(offsets), ptr(inputs), ptr(targets), i32(B),
                                         i32(sequence_length), i32(vocab_size)))
    return inputs, targets


def generate_batches_of_sequential_tokens(seed: int, *, vocab_size: int, sequence_length: int,
                                          global_batch_size_instances: int, total_batches: int,
                                          start_batch: int = 0, num_microbatches: int = 1, epoch: int = 0,
                                          device: str = "cuda") -> Iterator[List[Tuple[torch.Tensor, torch.Tensor]]]:
    """Yields, per batch, a list of `num_microbatches` (inputs, targets) pairs."""
    if global_batch_size_instances % num_microbatches != 0:
        raise ValueError("global batch size must be divisible by the number of micro-batches")
    per_mb = global_batch_size_instances // num_microbatches
    for batch_idx in range(start_batch, total_batches):
        batch = []
        for mb in range(num_microbatches):
            off = start_offsets(seed, epoch, batch_idx, mb, per_mb, vocab_size).to(device)
            batch.append(sequential_tokens(off, sequence_length, vocab_size))
        yield batch


class DataLoader:
    """Iterable over batches with the (key, batches_processed, epoch) state of the benchmark's loader."""

    def __init__(self, seed: int, *, vocab_size: int, sequence_length: int, global_batch_size_instances: int,
                 total_batches: int, num_microbatches: int = 1, device: str = "cuda"):
        self.seed, self.vocab_size, self.sequence_length = seed, vocab_size, sequence_length
        self.global_batch_size_instances, self.total_batches = global_batch_size_instances, total_batches
        self.num_microbatches, self.device = num_microbatches, device
        self.batches_processed = 0
        self.epoch = 0

    def __len__(self) -> int:
        return self.total_batches

    def __iter__(self):
        for batch in generate_batches_of_sequential_tokens(
                self.seed, vocab_size=self.vocab_size, sequence_length=self.sequence_length,
                global_batch_size_instances=self.global_batch_size_instances, total_batches=self.total_batches,
                start_batch=self.batches_processed, num_microbatches=self.num_microbatches, epoch=self.epoch,
                device=self.device):
            self.batches_processed += 1
            yield batch
        self.batches_processed = 0
        self.epoch += 1

    def get_state(self) -> Tuple[int, int, int]:
        return (self.seed, self.batches_processed, self.epoch)

    def load_state(self, state: Tuple[int, int, int]) -> None:
        self.seed, self.batches_processed, self.epoch = state
