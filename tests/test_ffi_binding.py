"""CPU-side checks of the JAX binding that ships as source (this image has no JAX): the adapter
TU only calls entry points the header declares, with as many arguments as the header gives them;
the Python module names a handler symbol for every target it registers; it fails with a clear
ImportError where JAX is missing; and the leaf table that maps the reference's pytree onto the
flat buffers packs and unpacks without loss."""
import importlib.util
import re
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = (ROOT / "include" / "olmax_hip.h").read_text()
ADAPTER = (ROOT / "olmax_amd" / "ffi" / "olmax_ffi.cc").read_text()


def _strip_comments(text):
    return re.sub(r"//[^\n]*", "", re.sub(r"/\*.*?\*/", "", text, flags=re.S))


def _split_args(s):
    out, depth, cur = [], 0, ""
    for ch in s:
        if ch in "([{":
            depth += 1
        elif ch in ")]}":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur)
            cur = ""
        else:
            cur += ch
    return [a for a in out + [cur] if a.strip() and a.strip() != "void"]


def _calls(text, name):
    """Argument lists of every call of `name(` in text (balanced parentheses)."""
    res = []
    for m in re.finditer(r"\b%s\s*\(" % re.escape(name), text):
        i, depth = m.end(), 1
        while depth:
            depth += {"(": 1, ")": -1}.get(text[i], 0)
            i += 1
        res.append(_split_args(text[m.end(): i - 1]))
    return res


def test_adapter_calls_match_the_header():
    header, adapter = _strip_comments(HEADER), _strip_comments(ADAPTER)
    called = sorted(set(re.findall(r"\b(olmax_[a-z0-9_]+)\s*\(", adapter)))
    assert {"olmax_attn_fwd", "olmax_attn_bwd", "olmax_rmsnorm_fwd", "olmax_rmsnorm_bwd", "olmax_gemm_bf16",
            "olmax_lmhead_ce", "olmax_adamw_dev", "olmax_model_train_step", "olmax_qk_rope_fwd", "olmax_qk_rope_bwd",
            "olmax_gemm_glu_bf16", "olmax_glu_bwd", "olmax_embed_fwd", "olmax_embed_bwd", "olmax_cross_entropy_reduce",
            "olmax_model_layout", "olmax_model_num_params", "olmax_model_workspace_bytes"} <= set(called)
    for name in called:
        decl = _calls(header, name)
        assert len(decl) == 1, f"{name} is not declared exactly once in olmax_hip.h"
        for args in _calls(adapter, name):
            assert len(args) == len(decl[0]), f"{name}: adapter passes {len(args)} arguments, header declares {len(decl[0])}"


def test_every_registered_target_has_a_handler_symbol():
    src = (ROOT / "olmax_amd" / "jax_ffi.py").read_text()
    targets = dict(re.findall(r'"(olmax_[a-z_]+)":\s*"(Olmax[A-Za-z]+)"', src))
    assert len(targets) == 16
    defined = set(re.findall(r"XLA_FFI_DEFINE_HANDLER_SYMBOL\(\s*(Olmax[A-Za-z]+)", ADAPTER))
    assert set(targets.values()) == defined
    used = set(re.findall(r'ffi_call\(\s*"(olmax_[a-z_]+)"', src))
    assert used == set(targets)


def test_jax_module_fails_clearly_without_jax():
    from olmax_amd import jax_ffi
    if importlib.util.find_spec("jax") is not None:
        pytest.skip("JAX is installed here")
    with pytest.raises(ImportError, match="needs jax"):
        jax_ffi.register()
    from olmax_amd import build
    assert build.xla_ffi_include_dir() is None and build.build_ffi_adapter() is None


def test_leaf_table_packs_the_reference_pytree_without_loss():
    from olmax_amd import _lib, TransformerConfig, layout
    if not _lib.lib_path().exists():
        pytest.skip("libolmax_hip.so not built")
    cfg = TransformerConfig(vocab_size=50, d_model=16, hidden_size=24, num_layers=2, n_heads=4, n_kv_heads=2, head_dim=8,
                            layer_type="gemma", qk_norm_headwise=True)
    table = layout.leaf_table(cfg)
    n = layout.num_params(cfg)
    names = [l.name for l in table]
    assert names[0] == "embedding.weight" and names[-1] == "lm_head.proj.weight" and "layers.1.mlp_input_norm.weight" in names
    by = {l.name: l for l in table}
    assert by["layers.0.attention.q_proj.weight"].shape == (32, 16) and by["layers.0.attention.k_proj.weight"].shape == (16, 16)
    assert by["layers.1.attention.q_norm.weight"].shape == (8,) and by["norm.weight"].shape == (16,)
    # q|k|v and gate|up are adjacent: each pair is one GEMM operand
    q, k, v = (by[f"layers.0.attention.{x}_proj.weight"] for x in "qkv")
    assert k.offset == q.offset + 32 * 16 and v.offset == k.offset + 16 * 16
    g, u = by["layers.1.mlp.gate_proj.weight"], by["layers.1.mlp.up_proj.weight"]
    assert u.offset == g.offset + 24 * 16
    rng = np.random.default_rng(0)
    named = {l.name: rng.normal(size=l.shape).astype(np.float32) for l in table}
    flat = np.full(n, np.nan, dtype=np.float32)
    layout.pack(cfg, named, flat)
    assert not np.isnan(flat).any()  # the leaves tile the buffer without gaps
    back = layout.unpack(cfg, flat)
    assert set(back) == set(named) and all(np.array_equal(back[k], named[k]) for k in named)
    with pytest.raises(KeyError):
        layout.pack(cfg, {k: v for k, v in named.items() if k != "norm.weight"}, flat)
    # full-width QK-norm changes the norm leaves' shapes only
    cfg2 = TransformerConfig(vocab_size=50, d_model=16, hidden_size=24, num_layers=1, n_heads=4, head_dim=8, qk_norm=True)
    by2 = {l.name: l for l in layout.leaf_table(cfg2)}
    assert by2["layers.0.attention.q_norm.weight"].shape == (32,) and by2["layers.0.attention.k_norm.weight"].shape == (32,)
