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
