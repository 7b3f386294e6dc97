"""CPU-side checks of the C-ABI boundary: the shared library loads and exports every symbol
that include/olmax_hip.h declares; host-only layout queries work without a GPU."""
import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def _declared():
    text = (ROOT / "include" / "olmax_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(olmax_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from olmax_amd import _lib
    if not _lib.lib_path().exists():
        pytest.skip("libolmax_hip.so not built (run `python -m olmax_amd.build`)")
    L = _lib.load()
    names = _declared()
    assert len(names) >= 30
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, missing
    assert L.olmax_abi_version() == 2


def test_layout_queries_on_host():
    from olmax_amd import _lib
    if not _lib.lib_path().exists():
        pytest.skip("libolmax_hip.so not built")
    from olmax_amd import TransformerRecipe
    from olmax_amd.transformer import CLeaf
    L = _lib.load()
    L.olmax_model_num_params.restype = ctypes.c_int64
    L.olmax_model_workspace_bytes.restype = ctypes.c_int64
    cfg = TransformerRecipe.llama_like_7B_bench()
    c = cfg.c_config(2, 4096)
    assert L.olmax_model_num_params(ctypes.byref(c)) == 7_298_355_200
    n = L.olmax_model_layout(ctypes.byref(c), None, 0)
    leaves = (CLeaf * n)()
    L.olmax_model_layout(ctypes.byref(c), leaves, n)
    # leaves tile the flat buffer without gaps or overlap
    spans = sorted((l.offset, l.offset + l.numel) for l in leaves)
    assert spans[0][0] == 0 and spans[-1][1] == 7_298_355_200
    assert all(a[1] == b[0] for a, b in zip(spans, spans[1:]))
    assert abs(cfg.flops_per_token(4096) / 1e9 - 44.544) < 1e-2
    # bad config is an error code, not a crash
    c.n_heads = 3
    c.n_kv_heads = 2
    assert L.olmax_model_num_params(ctypes.byref(c)) == -1
    assert b"multiple" in L.olmax_last_error_string()


def test_schedules_match_reference_known_answers():
    """src/test/optim/config_test.py:22-33."""
    from olmax_amd import WarmupCosineDecaySchedule, WarmupStableDecaySchedule
    s = WarmupStableDecaySchedule(warmup_steps=10, stable_steps=10, decay_steps=10, peak_value=1.0)
    r = [s(i) for i in range(31)]
    assert (r[0], r[5], r[10], r[20], r[25], r[30]) == (0.0, 0.5, 1.0, 1.0, 0.5, 0.0)
    c = WarmupCosineDecaySchedule(warmup_steps=20, decay_steps=80, peak_value=1e-4, init_value=1e-6, end_value=1e-6)
    assert c(0) == 1e-6 and abs(c(20) - 1e-4) < 1e-18 and abs(c(100) - 1e-6) < 1e-18


def test_ops_refuse_cpu_tensors():
    import torch
    from olmax_amd import _lib, ops
    with pytest.raises(_lib.OlmaxHipError):
        ops.rms_norm_fwd(torch.zeros(2, 8, dtype=torch.bfloat16), None, 1e-6)
