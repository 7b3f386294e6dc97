"""Optimizer configuration mirroring src/olmax/optim/config.py for the fused HIP AdamW."""
from __future__ import annotations

import fnmatch
import math
from dataclasses import dataclass, field
from typing import List, Optional


@dataclass
class ConstantSchedule:
    value: float = 0.0

    def __call__(self, step: int) -> float:
        return self.value


@dataclass
class WarmupCosineDecaySchedule:
    """src/olmax/optim/config.py:35-52 (optax.warmup_cosine_decay_schedule with
    decay_steps + warmup_steps passed as optax's total)."""
    warmup_steps: int
    decay_steps: int
    peak_value: float
    init_value: float = 0.0
    end_value: float = 0.0

    def __call__(self, step: int) -> float:
        if step < self.warmup_steps:
            return self.init_value + (self.peak_value - self.init_value) * step / max(1, self.warmup_steps)
        t = min(max(step - self.warmup_steps, 0), self.decay_steps)
        cos = 0.5 * (1.0 + math.cos(math.pi * t / max(1, self.decay_steps)))
        return self.end_value + (self.peak_value - self.end_value) * cos


@dataclass
class WarmupStableDecaySchedule:
    """src/olmax/optim/config.py:55-80."""
    warmup_steps: int
    stable_steps: int
    decay_steps: int
    peak_value: float
    init_value: float = 0.0
    end_value: float = 0.0

    def __call__(self, step: int) -> float:
        if step < self.warmup_steps:
            return self.init_value + (self.peak_value - self.init_value) * step / self.warmup_steps
        if step < self.warmup_steps + self.stable_steps:
            return self.peak_value
        t = min(step - self.warmup_steps - self.stable_steps, self.decay_steps)
        return self.peak_value + (self.end_value - self.peak_value) * t / self.decay_steps


@dataclass
class AdamWConfig:
    """src/olmax/optim/config.py:125-156.  ``no_decay_modules`` are fnmatch patterns over the
    dotted leaf paths (build_weight_decay_mask, config.py:94-122); the benchmark masks
    ``embedding.weight`` (src/integration_tests/train_transformer.py:388)."""
    lr: object = field(default_factory=lambda: ConstantSchedule(1e-4))
    b1: float = 0.9
    b2: float = 0.999
    eps: float = 1e-8
    weight_decay: float = 1e-4
    no_decay_modules: Optional[List[str]] = None
    max_grad_norm: Optional[float] = None

    def decays(self, name: str) -> bool:
        """Whether the leaf with this dotted path takes weight decay."""
        return not any(fnmatch.fnmatch(name, p) for p in (self.no_decay_modules or []))

    def lr_at(self, count: int) -> float:
        """Learning rate read at the pre-increment count (first step uses schedule(0))."""
        return float(self.lr(count)) if callable(self.lr) else float(self.lr)
