"""The train step of src/olmax/train/trainer.py:759-777 (process_microbatch) on the HIP path."""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

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

    def train_batch(self, batch: Sequence[Tuple[torch.Tensor, torch.Tensor]]) -> torch.Tensor:
        """train_batch (reference src/olmax/train/trainer.py:779-807): one micro-batch at a time.
        With one micro-batch this is process_microbatch.  With k > 1 the optimizer is wrapped in
        optax.MultiSteps(k) (src/olmax/optim/config.py:153-154): each micro-batch's gradients
        enter a running fp32 mean, the AdamW update (with the clip, on the mean) is applied after
        the last one, and the schedule advances once per batch.  Returns the mean of the
        micro-batch losses (trainer.py:796)."""
        k = len(batch)
        if k == 0:
            raise ValueError("train_batch: empty batch")
        if k == 1:
            return self.process_microbatch(*batch[0])
        lr = self.optim.lr_at(self.count)
        self.count += 1
        losses = []
        for j, (ids, labels) in enumerate(batch):
            losses.append(self.model.loss_and_grads(ids, labels).clone())
            self.model.accumulate_grads(j)
        self.model.adamw_step_accumulated(step=self.count, lr=lr, b1=self.optim.b1, b2=self.optim.b2, eps=self.optim.eps,
                                          weight_decay=self.optim.weight_decay, decay_embedding=self._decay_embedding,
                                          max_grad_norm=self.optim.max_grad_norm)
        return torch.stack(losses).mean()

    @property
    def grad_norm(self) -> Optional[float]:
        if self.optim.max_grad_norm is None:
            return None
        return float(self.model.norm_scratch[1].item())
