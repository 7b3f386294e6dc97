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


def test_adapter_type_checks_against_a_model_of_the_xla_ffi_api():
    """The adapter cannot be built here (the XLA headers ship inside jaxlib), but it can be
    type-checked: tests/xla_ffi_model holds a minimal model of the API in which every
    XLA_FFI_DEFINE_HANDLER_SYMBOL asserts that the handler accepts exactly the parameter list its
    Ctx / Arg / Ret / Attr chain describes.  -fsyntax-only: nothing is built or run."""
    import shutil
    import subprocess
    gxx = shutil.which("g++")
    if gxx is None or not Path("/opt/rocm/include/hip/hip_runtime_api.h").exists():
        pytest.skip("needs g++ and the HIP headers")
    cmd = [gxx, "-std=c++17", "-fsyntax-only", "-Wall", "-Werror", "-D__HIP_PLATFORM_AMD__", "-I", str(ROOT / "tests" / "xla_ffi_model"),
           "-I", str(ROOT / "include"), "-I", "/opt/rocm/include"]
    r = subprocess.run(cmd + [str(ROOT / "olmax_amd" / "ffi" / "olmax_ffi.cc")], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    # the model does reject a handler whose binding lost an attribute
    bad = ADAPTER.replace('.Attr<int32_t>("window").Attr<float>("softcap"));', '.Attr<int32_t>("window"));', 1)
    assert bad != ADAPTER
    r = subprocess.run(cmd + ["-I", str(ROOT / "olmax_amd" / "ffi"), "-x", "c++", "-"], input=bad, capture_output=True, text=True)
    assert r.returncode != 0 and "do not match" in r.stderr


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


# ----------------------------------------------------------------------------------------------
# The Python half of the binding, run against a numpy-backed model of the JAX API (tests/jax_model):
# every wrapper and both rules of every custom_vjp execute, and each custom call they make is compared
# with the handler binding of the same target in the adapter.
# ----------------------------------------------------------------------------------------------
def _handler_bindings():
    out = {}
    for m in re.finditer(r"XLA_FFI_DEFINE_HANDLER_SYMBOL\(\s*(Olmax\w+)\s*,\s*\w+\s*,(.*?)\)\s*;", _strip_comments(ADAPTER), re.S):
        sym, chain = m.groups()
        out[sym] = dict(args=chain.count(".Arg<"), rets=chain.count(".Ret<"), attrs=dict((n, t) for t, n in re.findall(r'\.Attr<(\w+)>\("(\w+)"\)', chain)))
    return out


@pytest.fixture
def jax_model(monkeypatch):
    import sys
    if importlib.util.find_spec("jax") is not None:
        pytest.skip("JAX is installed here: the model is for machines without it")
    from olmax_amd import _lib, jax_ffi
    if not _lib.lib_path().exists():
        pytest.skip("libolmax_hip.so not built (the wrappers ask it for workspace sizes)")
    monkeypatch.syspath_prepend(str(ROOT / "tests" / "jax_model"))
    caches = [getattr(jax_ffi, n) for n in dir(jax_ffi) if n.endswith("_vjp") and hasattr(getattr(jax_ffi, n), "cache_clear")]
    for c in caches:
        c.cache_clear()
    import jax
    jax.ffi.CALLS.clear()
    monkeypatch.setattr(jax_ffi, "register", lambda lib_path=None: None)
    yield jax
    for c in caches:
        c.cache_clear()
    for name in [n for n in sys.modules if n == "jax" or n.startswith("jax.") or n == "optax"]:
        del sys.modules[name]


def _check_calls(jax, expected_targets):
    from olmax_amd import jax_ffi
    bindings = _handler_bindings()
    assert len(bindings) == 16
    seen = [c["target"] for c in jax.ffi.CALLS]
    assert seen == expected_targets, seen
    for c in jax.ffi.CALLS:
        b = bindings[jax_ffi._TARGETS[c["target"]]]
        assert len(c["operands"]) == b["args"], f'{c["target"]}: {len(c["operands"])} operands, the handler binds {b["args"]}'
        assert len(c["results"]) == b["rets"], f'{c["target"]}: {len(c["results"])} results, the handler binds {b["rets"]}'
        assert set(c["attrs"]) == set(b["attrs"]), f'{c["target"]}: attributes {sorted(c["attrs"])} vs {sorted(b["attrs"])}'
        for name, ctype in b["attrs"].items():
            v = c["attrs"][name]
            if ctype == "int32_t":
                assert isinstance(v, np.int32), (c["target"], name, type(v))
            elif ctype == "float":
                assert isinstance(v, np.float32), (c["target"], name, type(v))
            else:
                assert ctype == "I32s" and isinstance(v, np.ndarray) and v.dtype == np.int32 and v.ndim == 1, (c["target"], name)
        for i, o in c["aliases"].items():
            assert c["operands"][i].shape == c["results"][o].shape and c["operands"][i].dtype == c["results"][o].dtype
    jax.ffi.CALLS.clear()


def test_wrappers_and_vjp_rules_make_the_calls_the_handlers_bind(jax_model):
    jax = jax_model
    jnp = jax.numpy
    from olmax_amd import jax_ffi
    BF = jnp.bfloat16
    B, S, H, K, D, d, F, V = 2, 8, 4, 2, 16, 32, 48, 64
    q, k, v = np.zeros((B, S, H, D), BF), np.zeros((B, S, K, D), BF), np.zeros((B, S, K, D), BF)
    # attention: forward, then both rules
    o = jax_ffi.hip_attention(q, k, v, window=3, softcap=50.0)
    assert o.shape == q.shape and o.dtype == q.dtype
    _, (dq, dk, dv) = jax_ffi._attention_vjp().run_vjp(q, k, v, 3, 50.0)
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    _check_calls(jax, ["olmax_attn_fwd", "olmax_attn_fwd", "olmax_attn_bwd"])
    # rms_norm
    x, w = np.zeros((B, S, d), BF), np.ones((d,), BF)
    assert jax_ffi.hip_rms_norm(x, w, 1e-6).shape == x.shape
    _, (dx, dw) = jax_ffi._rms_norm_vjp().run_vjp(x, w, 1e-6)
    assert dx.shape == x.shape and dw.shape == w.shape and dw.dtype == w.dtype
    _check_calls(jax, ["olmax_rmsnorm_fwd", "olmax_rmsnorm_fwd", "olmax_rmsnorm_bwd"])
    # linear: y = x W^T and its two transposes
    W = np.zeros((F, d), BF)
    y = jax_ffi.hip_linear(x, W)
    assert y.shape == (B, S, F)
    _, (dx, dW) = jax_ffi._linear_vjp().run_vjp(x, W)
    assert dx.shape == x.shape and dW.shape == W.shape
    _check_calls(jax, ["olmax_gemm"] * 4)
    # LM head + cross entropy: labels are an array argument without cotangent
    Wv, labels = np.zeros((V, d), BF), np.zeros((B, S), np.int64)
    loss = jax_ffi.hip_lm_head_cross_entropy(x, Wv, labels, 30.0)
    assert loss.shape == ()
    _, (dh, dWv, dlab) = jax_ffi._lm_head_vjp().run_vjp(x, Wv, labels, 30.0)
    assert dh.shape == x.shape and dWv.shape == Wv.shape and dlab is None
    assert all(c["operands"][2].dtype == np.int32 and c["operands"][2].ndim == 1 for c in jax.ffi.CALLS)
    _check_calls(jax, ["olmax_lmhead_ce"] * 2)
    # cross entropy on logits, the three reductions
    logits = np.zeros((B, S, V), np.float32)
    for red in ("mean", "sum", "none"):
        loss, lse = jax_ffi.hip_fused_cross_entropy_loss(logits, labels, reduction=red)
        assert loss.shape == ((B, S) if red == "none" else ()) and lse.shape == (B, S, 1)
        (_, _), (dz, dlab) = jax_ffi._cross_entropy_vjp().run_vjp(logits, labels, -100, jax_ffi._REDUCTIONS[red], 0.0)
        assert dz.shape == logits.shape and dlab is None
        _check_calls(jax, ["olmax_cross_entropy_fwd", "olmax_cross_entropy_fwd", "olmax_cross_entropy_bwd"])
    assert jax_ffi.hip_cross_entropy_loss(logits, labels).shape == ()
    jax.ffi.CALLS.clear()
    # RoPE with and without the head-wise norm
    cos, sin = np.ones((S, D // 2), np.float32), np.zeros((S, D // 2), np.float32)
    assert jax_ffi.hip_rope(q, cos, sin).shape == q.shape
    assert jax_ffi.hip_rope(q, cos, sin, norm_weight=np.ones((D,), BF), eps=1e-6).shape == q.shape
    _, grads = jax_ffi._rope_vjp().run_vjp(q, np.ones((D,), BF), cos, sin, True, 1e-6)
    assert grads[0].shape == q.shape and grads[1].shape == (D,) and grads[2].shape == cos.shape and grads[3].shape == sin.shape
    _check_calls(jax, ["olmax_qk_rope_fwd"] * 3 + ["olmax_qk_rope_bwd"])
    # gated MLP input half
    Wg, Wu = np.zeros((F, d), BF), np.zeros((F, d), BF)
    assert jax_ffi.hip_gated_mlp_in(x, Wg, Wu, "gelu").shape == (B, S, F)
    _, (dx, dWg, dWu) = jax_ffi._gated_vjp().run_vjp(x, Wg, Wu, 1)
    assert dx.shape == x.shape and dWg.shape == Wg.shape and dWu.shape == Wu.shape
    _check_calls(jax, ["olmax_gemm_glu", "olmax_gemm_glu", "olmax_glu_bwd", "olmax_gemm", "olmax_gemm"])
    # embedding
    E, ids = np.zeros((V, d), BF), np.zeros((B, S), np.int64)
    assert jax_ffi.hip_embedding(E, ids).shape == (B, S, d)
    _, (dE, dids) = jax_ffi._embedding_vjp().run_vjp(E, ids)
    assert dE.shape == E.shape and dE.dtype == E.dtype and dids is None
    assert all(c["operands"][0].dtype == np.int32 for c in jax.ffi.CALLS)
    _check_calls(jax, ["olmax_embed_fwd", "olmax_embed_fwd", "olmax_embed_bwd"])


def test_adamw_transformation_and_train_step_make_the_calls_the_handlers_bind(jax_model):
    jax = jax_model
    from olmax_amd import TransformerConfig, jax_ffi, layout
    # optax-style transformation: one custom call per leaf, state (count, mu, nu), updates = p_new - p
    params = {"a": np.ones((4, 8), np.float32), "b": {"w": np.ones((8,), np.float32)}}
    grads = jax.tree.map(np.zeros_like, params)
    tx = jax_ffi.hip_adamw(lambda count: 1e-3, weight_decay=0.1, mask={"a": True, "b": {"w": False}})
    state = tx.init(params)
    updates, state2 = tx.update(grads, state, params)
    assert set(updates) == {"a", "b"} and updates["a"].shape == (4, 8) and int(state2[0]) == 1
    wds = sorted(float(c["attrs"]["wd"]) for c in jax.ffi.CALLS)
    assert wds == [0.0, pytest.approx(0.1)]
    assert all(c["operands"][4].shape == (3,) and c["operands"][4].dtype == np.float32 for c in jax.ffi.CALLS)
    _check_calls(jax, ["olmax_adamw"] * 2)
    # the whole step: attribute vector, table selection and buffer sizes follow the layout
    cfg = TransformerConfig(vocab_size=64, d_model=32, hidden_size=48, num_layers=3, n_heads=4, n_kv_heads=2, head_dim=8,
                            layer_type="gemma", qk_norm_headwise=True, window_size_per_layer=[4, None, 4],
                            rope_theta_per_layer=[1e4, 1e6, 1e4])
    B, S = 2, 16
    step = jax_ffi.HipTrainStep(cfg, batch_size=B, sequence_length=S, learning_rate=lambda c: 1e-4, weight_decay=0.1,
                                no_decay_modules=["embedding.weight"])
    n = layout.num_params(cfg)
    named = {l.name: np.zeros(l.shape, np.float32) for l in step.table}
    flat = np.concatenate([named[l.name].reshape(-1) for l in step.table])
    assert flat.shape == (n,)
    state = (flat, np.zeros_like(flat), np.zeros_like(flat), flat.astype(jax.numpy.bfloat16))
    new_state, loss, norm = step(state, np.zeros((B, S), np.int64), np.zeros((B, S), np.int64), np.zeros([], np.int32))
    assert len(new_state) == 4 and loss.shape == () and norm.shape == (2,)
    call = jax.ffi.CALLS[0]
    assert call["attrs"]["config"].shape == (14,) and len(call["attrs"]["windows"]) == 3
    assert list(call["attrs"]["table_index"]) == [0, 1, 0] and step.cos.shape == (2, S, 4)
    decay = list(call["attrs"]["leaf_decay"])
    assert len(decay) == len(step.table) and decay[0] == 0 and sum(decay) == len(decay) - 1
    assert call["operands"][4].dtype == np.int32 and call["operands"][4].shape == (B * S,)
    assert call["operands"][8].shape == (3,) and call["results"][6].shape == (step.nf,) and call["results"][7].shape == (step.ws_bytes,)
    _check_calls(jax, ["olmax_train_step"])
    back = step.unpack(new_state)
    assert set(back) == set(named) and all(back[k].shape == named[k].shape for k in named)
