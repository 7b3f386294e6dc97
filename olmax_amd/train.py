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

    # ------------------------------------------------------------------ checkpoint
    def save_checkpoint(self, path: str, data_loader=None, tokens_seen: Optional[int] = None) -> None:
        """Write the train state the reference keeps in TrainState (src/olmax/train/trainer.py:45-53:
        step, tokens seen, params, optimizer state, data-loader state) to one safetensors file:
        the flat fp32 master parameters and both Adam moments as three tensors, everything else
        as string metadata.  (The reference's orbax directory format is not reproduced.)"""
        import json

        from safetensors.torch import save_file

        m = self.model
        if m.m is None:
            m.init_optimizer_state()
        meta = {"format": "olmax_amd.train_state.v1", "step": str(self.count), "num_params": str(m.num_params),
                "tokens_seen": json.dumps(tokens_seen),
                "data_loader_state": json.dumps(None if data_loader is None else list(data_loader.get_state()))}
        torch.cuda.synchronize()
        save_file({"master": m.master, "adam_m": m.m, "adam_v": m.v}, path, metadata=meta)

    def load_checkpoint(self, path: str, data_loader=None) -> dict:
        """Restore what save_checkpoint wrote; the bf16 working copy is rebuilt from the master
        parameters.  Returns the metadata (step, tokens_seen, data_loader_state)."""
        import json

        from safetensors import safe_open

        m = self.model
        if m.m is None:
            m.init_optimizer_state()
        with safe_open(path, framework="pt", device="cpu") as f:
            meta = f.metadata() or {}
            if meta.get("format") != "olmax_amd.train_state.v1":
                raise ValueError(f"{path}: not an olmax_amd train state")
            if int(meta["num_params"]) != m.num_params:
                raise ValueError(f"{path}: holds {meta['num_params']} parameters, the model has {m.num_params}")
            for name, dst in (("master", m.master), ("adam_m", m.m), ("adam_v", m.v)):
                dst.copy_(f.get_tensor(name))
        m.sync_working_copy()
        self.count = int(meta["step"])
        state = json.loads(meta["data_loader_state"])
        if data_loader is not None and state is not None:
            data_loader.load_state(tuple(state))
        return {"step": self.count, "tokens_seen": json.loads(meta["tokens_seen"]), "data_loader_state": state}

    @staticmethod
    def set_profiler_ranges(on: bool) -> None:
        """roctx ranges per layer and phase from the whole-model entry points (the counterpart of
        the reference's named scopes, src/olmax/train/callbacks/profiler.py:33-50)."""
        from ._lib import check, i32, load

        check(load().olmax_set_profiler_ranges(i32(int(on))))

    @property
    def grad_norm(self) -> Optional[float]:
        if self.optim.max_grad_norm is None:
            return None
        return float(self.model.norm_scratch[1].item())
