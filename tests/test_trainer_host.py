"""Host-side trainer logic that needs no GPU: the running statistics and the throughput metrics
(reference src/olmax/utils.py:209-246, src/olmax/train/trainer.py:596-627) and the NaN-loss check
made when a step's metrics are logged (src/olmax/train/trainer.py:706-710)."""
import math

import numpy as np
import pytest

from olmax_amd.train import RunningAverage, ThroughputMeter, Trainer


def test_running_average_matches_numpy():
    rng = np.random.default_rng(0)
    x = rng.normal(3.0, 2.0, size=257)
    ra = RunningAverage()
    with pytest.raises(ZeroDivisionError):
        ra.get()
    for i, v in enumerate(x, 1):
        assert ra.update(float(v)) == pytest.approx(x[:i].mean(), rel=1e-12, abs=1e-12)
        if i == 1:
            with pytest.raises(ZeroDivisionError):
                ra.get_variance()
    assert ra.count == 257
    assert ra.get_variance() == pytest.approx(x.var(), rel=1e-10)
    assert ra.get_sample_variance() == pytest.approx(x.var(ddof=1), rel=1e-10)
    ra.reset()
    assert ra.count == 0 and ra.mean == 0.0


def test_throughput_metrics_thresholds_and_formulas():
    """Instantaneous rates every step; averages only from the 10th step of the run; the standard
    deviation once the average holds five samples, i.e. from the 14th step."""
    m = ThroughputMeter()
    secs = [0.5 + 0.01 * i for i in range(20)]
    tokens = 8192
    seen = []
    for step, dt in enumerate(secs, 1):
        out = m.update(step, dt, tokens)
        assert out["throughput/BPS"] == pytest.approx(1.0 / dt)
        assert out["throughput/TPS"] == pytest.approx(tokens / dt)
        assert out["throughput/TPS device"] == out["throughput/TPS"]
        assert ("throughput/BPS average" in out) == (step >= 10)
        assert ("throughput/BPS stddev" in out) == (step >= 14)
        if step >= 10:
            seen.append(1.0 / dt)
            assert out["throughput/BPS average"] == pytest.approx(np.mean(seen))
            assert out["throughput/TPS average"] == pytest.approx(np.mean(seen) * tokens)
        if step >= 14:
            assert out["throughput/BPS stddev"] == pytest.approx(np.std(seen, ddof=1))
            assert out["throughput/TPS stddev"] == pytest.approx(np.std(seen, ddof=1) * tokens)
    # without a token count only the batch rates are reported
    assert set(ThroughputMeter().update(1, 0.25, None)) == {"throughput/BPS"}


def test_logging_order_exclusion_and_nan_loss():
    tr = Trainer.__new__(Trainer)  # host logic only: no model, no GPU
    tr.count = 1
    tr.record_metric("train/loss", 2.5)
    tr.count = 2
    tr.record_metric("train/loss", 2.25)
    tr.record_metric("optim/lr", 1e-3)
    logged = []
    tr._log_metrics(lambda s, m: logged.append((s, m)), exclude=2)
    assert logged == [(1, {"train/loss": 2.5})]
    tr._log_metrics(lambda s, m: logged.append((s, m)))
    assert logged[1] == (2, {"train/loss": 2.25, "optim/lr": 1e-3}) and tr._metrics == {}
    tr.count = 3
    tr.record_metric("train/loss", math.nan)
    with pytest.raises(RuntimeError, match="step 3"):
        tr._log_metrics(None)


def test_fit_stops_before_pulling_a_batch_it_will_not_train_on(monkeypatch):
    """The loop tests completion BEFORE it asks the loader for the next batch (reference
    src/olmax/train/trainer.py:522-551), so that a loader state saved after fit() points at the first
    batch that was NOT trained on; a loader that runs dry ends the loop as well."""
    import torch

    from olmax_amd.optim import AdamWConfig, ConstantSchedule

    class CountingLoader:
        def __init__(self, n):
            self.n, self.batches_processed = n, 0

        def __iter__(self):
            while self.batches_processed < self.n:
                self.batches_processed += 1  # counted when handed out, as data.DataLoader does
                yield [(torch.zeros(4, dtype=torch.int32), torch.zeros(4, dtype=torch.int32))]

        def get_state(self):
            return (0, self.batches_processed, 0)

    monkeypatch.setattr(torch.cuda, "synchronize", lambda *a, **k: None)
    tr = Trainer.__new__(Trainer)  # host logic only: the step itself is replaced
    tr.count, tr.optim = 0, AdamWConfig(lr=ConstantSchedule(1e-3))

    def fake_train_batch(batch):
        tr.count += 1
        return 1.0 / tr.count

    tr.train_batch = fake_train_batch
    dl = CountingLoader(10)
    logged = []
    tr.fit(dl, max_steps=4, log_fn=lambda s, m: logged.append(s))
    assert tr.count == 4 and dl.get_state()[1] == 4 and logged == [1, 2, 3, 4]
    tr.fit(dl, max_steps=4)   # already complete: nothing is pulled
    assert dl.get_state()[1] == 4
    tr.fit(dl, max_steps=100)  # the loader runs dry after 6 more
    assert tr.count == 10 and dl.get_state()[1] == 10


def test_adamw_config_decay_patterns():
    """fnmatch patterns over dotted leaf paths (src/olmax/optim/config.py:94-122; the reference's own
    mask test, src/test/optim/config_test.py:36-47, on its names)."""
    from olmax_amd.optim import AdamWConfig

    c = AdamWConfig(no_decay_modules=["gate_proj.bias", "down_proj.bias", "up_proj.bias"])
    for m in ("gate_proj", "down_proj", "up_proj"):
        assert c.decays(f"{m}.weight") is True and c.decays(f"{m}.bias") is False
    c = AdamWConfig(no_decay_modules=["embedding.weight", "*norm.weight"])
    assert not c.decays("embedding.weight") and not c.decays("layers.3.attention.q_norm.weight") and not c.decays("norm.weight")
    assert c.decays("layers.3.mlp.up_proj.weight") and c.decays("lm_head.proj.weight")
    assert AdamWConfig().decays("embedding.weight")
