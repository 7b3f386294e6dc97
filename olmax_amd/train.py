"""The train step of src/olmax/train/trainer.py:759-777 (process_microbatch) on the HIP path."""
from __future__ import annotations

from typing import Optional

import torch

from .optim import AdamWConfig
from .transformer import Transformer


class Trainer:
    """Minimal step driver: loss + grads, then the fused AdamW update, once per micro-batch."""

    def __init__(self, model: Transformer, optim: AdamWConfig, overlap_optimizer: bool = True):
        self.model, self.optim = model, optim
        self.overlap_optimizer = overlap_optimizer
        self.count = 0  # optimizer steps taken
        self._decay_embedding = optim.decay_embedding()
        model.init_optimizer_state()

    def process_microbatch(self, input_ids: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
        lr = self.optim.lr_at(self.count)
        self.count += 1
        return self.model.train_step(input_ids, labels, step=self.count, lr=lr, b1=self.optim.b1, b2=self.optim.b2,
                                     eps=self.optim.eps, weight_decay=self.optim.weight_decay,
                                     decay_embedding=self._decay_embedding, max_grad_norm=self.optim.max_grad_norm,
                                     overlap_optimizer=self.overlap_optimizer)

    @property
    def grad_norm(self) -> Optional[float]:
        if self.optim.max_grad_norm is None:
            return None
        return float(self.model.norm_scratch[1].item())
