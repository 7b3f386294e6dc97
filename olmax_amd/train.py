"""The train step of src/olmax/train/trainer.py:759-777 (process_microbatch) on the HIP path."""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import torch

from .optim import AdamWConfig
from .transformer import Transformer


class RunningAverage:
    """Online mean and variance (Welford), the statistic behind the reference's averaged
    throughput metrics (src/olmax/utils.py:209-246)."""

    def __init__(self) -> None:
        self.reset()

    def reset(self) -> None:
        self.mean, self.m2, self.count = 0.0, 0.0, 0

    def update(self, value: float) -> float:
        self.count += 1
        d = value - self.mean
        self.mean += d / self.count
        self.m2 += d * (value - self.mean)
        return self.mean

    def get(self) -> float:
        if self.count == 0:
            raise ZeroDivisionError("no samples")
        return self.mean

    def get_variance(self) -> float:
        if self.count < 2:
            raise ZeroDivisionError("variance needs two samples")
        return self.m2 / self.count

    def get_sample_variance(self) -> float:
        if self.count < 2:
            raise ZeroDivisionError("variance needs two samples")
        return self.m2 / (self.count - 1)


class ThroughputMeter:
    """Batches and tokens per second as the reference reports them (src/olmax/train/trainer.py:596-627):
    the instantaneous rate every step; the running average from the 10th step of a run on (the first
    steps carry compilation and warm-up there); the sample standard deviation once the average holds
    5 samples.  One GPU: the per-device figures equal the global ones."""

    def __init__(self, n_devices: int = 1) -> None:
        self.avg = RunningAverage()
        self.n_devices = n_devices

    def update(self, step_this_run: int, seconds: float, tokens_this_batch: Optional[int]) -> dict:
        import math

        bps = 1.0 / seconds
        bps_avg = None if step_this_run < 10 else self.avg.update(bps)
        bps_std = None if self.avg.count < 5 else math.sqrt(self.avg.get_sample_variance())
        out = {"throughput/BPS": bps}
        if bps_avg is not None:
            out["throughput/BPS average"] = bps_avg
        if bps_std is not None:
            out["throughput/BPS stddev"] = bps_std
        if tokens_this_batch is not None:
            out["throughput/TPS"] = bps * tokens_this_batch
            out["throughput/TPS device"] = out["throughput/TPS"] / self.n_devices
            if bps_avg is not None:
                out["throughput/TPS average"] = bps_avg * tokens_this_batch
                out["throughput/TPS device average"] = out["throughput/TPS average"] / self.n_devices
            if bps_std is not None:
                out["throughput/TPS stddev"] = bps_std * tokens_this_batch
                out["throughput/TPS device stddev"] = out["throughput/TPS stddev"] / self.n_devices
        return out


class Trainer:
    """Minimal step driver: loss + grads, then the fused AdamW update, once per micro-batch."""

    def __init__(self, model: Transformer, optim: AdamWConfig, overlap_optimizer: bool = True):
        self.model, self.optim = model, optim
        self.overlap_optimizer = overlap_optimizer
        self.count = 0  # optimizer steps taken
        self._no_decay = tuple(optim.no_decay_modules or ())
        model.weight_decay_mask(self._no_decay)  # warns now about patterns that match nothing
        model.init_optimizer_state()

    def process_microbatch(self, input_ids: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
        lr = self.optim.lr_at(self.count)
        self.count += 1
        return self.model.train_step(input_ids, labels, step=self.count, lr=lr, b1=self.optim.b1, b2=self.optim.b2,
                                     eps=self.optim.eps, weight_decay=self.optim.weight_decay,
                                     no_decay_modules=self._no_decay, max_grad_norm=self.optim.max_grad_norm,
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
                                          weight_decay=self.optim.weight_decay, no_decay_modules=self._no_decay,
                                          max_grad_norm=self.optim.max_grad_norm)
        return torch.stack(losses).mean()

    # ------------------------------------------------------------------ metrics and the training loop
    def record_metric(self, name: str, value) -> None:
        """Queue a metric of the current step (reference record_metric, src/olmax/train/trainer.py:274-278).
        A device scalar starts its copy to pinned host memory on the current stream and is only read
        when the step is logged, one step later, so logging never drains the GPU queue."""
        if not hasattr(self, "_metrics"):
            self._metrics = {}
        if isinstance(value, torch.Tensor) and value.is_cuda:
            host = torch.empty((), dtype=value.dtype, pin_memory=True)
            host.copy_(value.detach().reshape(()), non_blocking=True)
            ev = torch.cuda.Event()
            ev.record()
            value = (host, ev)
        self._metrics.setdefault(self.count, {})[name] = value

    def _log_metrics(self, log_fn, exclude: Optional[int] = None) -> None:
        import math

        for step in sorted(getattr(self, "_metrics", {})):
            if step == exclude:
                continue
            out = {}
            for name, v in self._metrics.pop(step).items():
                if isinstance(v, tuple):
                    v[1].synchronize()
                    v = float(v[0])
                out[name] = float(v)
            if log_fn is not None:
                log_fn(step, out)
            loss = out.get("train/loss")
            if loss is not None and not math.isfinite(loss):
                raise RuntimeError(f"NaN loss encountered on step {step}!")

    def fit(self, data_loader, max_steps: int, log_fn=None, tokens_per_batch: Optional[int] = None) -> None:
        """The reference's training loop (src/olmax/train/trainer.py:531-637) on one GPU.  Every item
        of `data_loader` is one batch, a list of (input_ids, labels) micro-batches as
        data.DataLoader yields them.  Per step: train on the batch, queue train/loss, optim/lr and
        (when clipping) optim/g_norm, hand the metrics of earlier steps to `log_fn(step, dict)`
        while this step still runs on the GPU, and record batches and tokens per second."""
        import time

        meter = ThroughputMeter()
        step_this_run = 0
        t0 = time.perf_counter()
        batches = iter(data_loader)
        while self.count < max_steps:  # tested BEFORE the next batch is pulled (trainer.py:522-551):
            try:                       # the loader state stays at what was trained on
                batch = next(batches)
            except StopIteration:
                break
            step_this_run += 1
            tokens = tokens_per_batch if tokens_per_batch is not None else sum(int(ids.numel()) for ids, _ in batch)
            lr = self.optim.lr_at(self.count)  # read before the count moves: the first step uses schedule(0)
            loss = self.train_batch([(ids.reshape(-1), labels.reshape(-1)) for ids, labels in batch])
            self.record_metric("train/loss", loss)
            self.record_metric("optim/lr", lr)
            if self.optim.max_grad_norm is not None:
                self.record_metric("optim/g_norm", self.model.norm_scratch[1])
            self._log_metrics(log_fn, exclude=self.count)
            t1 = time.perf_counter()
            for name, v in meter.update(step_this_run, t1 - t0, tokens).items():
                self.record_metric(name, v)
            t0 = t1
        torch.cuda.synchronize()
        self._log_metrics(log_fn)

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
