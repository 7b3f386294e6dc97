"""JAX side of the drop-in: libolmax_hip's entry points as jax.ffi custom calls.

What a maintainer of the reference adds to run its Equinox modules and trainer on the HIP path
(the reference itself has no FFI seam; these are the three places its kernels are chosen):

* ``hip_attention``      for ``AttentionKernel.forward`` (src/olmax/nn/attention.py:64-103), behind a new
                         ``implementation="hip"`` literal;
* ``hip_rms_norm``, ``hip_linear``, ``hip_lm_head_cross_entropy`` for the pure functions of
                         src/olmax/nn/functional.py:21,51,70 (+ ``LMHead.forward``, lm_head.py:59-61);
* ``hip_cross_entropy_loss`` / ``hip_fused_cross_entropy_loss`` for src/olmax/nn/functional.py:70-121 on given
                         logits (all three reductions; the fused one also returns the log-normaliser);
* ``hip_rope``           for ``RotaryPositionalEmbedding.forward`` (src/olmax/nn/rope.py:68-80), optionally with the
                         head-wise QK-norm of src/olmax/nn/attention.py:293-296 folded in;
* ``hip_gated_mlp_in``   for the gate / up half of ``GatedMLP.forward`` (src/olmax/nn/mlp.py:69-73): one GEMM with the
                         activation in its epilogue;
* ``hip_embedding``      for ``Embedding.forward`` (src/olmax/nn/embedding.py:30-32);
* ``hip_adamw``          an ``optax.GradientTransformation`` for ``optim.update`` at
                         src/olmax/train/trainer.py:745;
* ``HipTrainStep``       ``process_microbatch`` (src/olmax/train/trainer.py:759-777) as ONE custom call on
                         flat, donated buffers: the granularity ``bench.py`` measures.

Every differentiable op is a ``jax.custom_vjp`` whose backward is a second custom call (JAX cannot
differentiate through an FFI call).  Nothing here computes: the handlers of ``ffi/olmax_ffi.cc``
unpack buffers and call the C ABI.  JAX is imported lazily: this image has no JAX, so the module
is committed as source and exercised only where jaxlib (and its XLA FFI headers, needed to build
``libolmax_ffi.so``, see ``olmax_amd.build.build_ffi_adapter``) exists.
"""
from __future__ import annotations

import ctypes
import functools
from pathlib import Path
from typing import Optional, Sequence

import numpy as np

from . import _lib

FFI_LIB = Path(__file__).resolve().parent / "libolmax_ffi.so"
_TARGETS = {"olmax_attn_fwd": "OlmaxAttnFwd", "olmax_attn_bwd": "OlmaxAttnBwd", "olmax_rmsnorm_fwd": "OlmaxRmsNormFwd",
            "olmax_rmsnorm_bwd": "OlmaxRmsNormBwd", "olmax_gemm": "OlmaxGemm", "olmax_lmhead_ce": "OlmaxLmHeadCe",
            "olmax_adamw": "OlmaxAdamW", "olmax_train_step": "OlmaxTrainStep",
            "olmax_qk_rope_fwd": "OlmaxQkRopeFwd", "olmax_qk_rope_bwd": "OlmaxQkRopeBwd", "olmax_gemm_glu": "OlmaxGemmGlu",
            "olmax_glu_bwd": "OlmaxGluBwd", "olmax_embed_fwd": "OlmaxEmbedFwd", "olmax_embed_bwd": "OlmaxEmbedBwd",
            "olmax_cross_entropy_fwd": "OlmaxCrossEntropyFwd", "olmax_cross_entropy_bwd": "OlmaxCrossEntropyBwd"}
_registered = False


def _jax():
    try:
        import jax
        import jax.numpy as jnp
    except ImportError as e:  # pragma: no cover - this image has no JAX
        raise ImportError("olmax_amd.jax_ffi needs jax/jaxlib (ROCm build); it is not installed here") from e
    return jax, jnp


def register(lib_path: Optional[str] = None) -> None:
    """Load libolmax_ffi.so and register every handler for platform "ROCM" (idempotent)."""
    global _registered
    jax, _ = _jax()
    if _registered:
        return
    path = Path(lib_path) if lib_path else FFI_LIB
    if not path.exists():
        raise _lib.OlmaxHipError(f"{path} not found: build it with olmax_amd.build.build_ffi_adapter() "
                                 "(needs the XLA FFI headers of jaxlib)")
    _lib.load()  # libolmax_hip.so first: the adapter links against it
    lib = ctypes.CDLL(str(path))
    for target, symbol in _TARGETS.items():
        jax.ffi.register_ffi_target(target, jax.ffi.pycapsule(getattr(lib, symbol)), platform="ROCM")
    _registered = True


def _sds(shape, dtype):
    jax, _ = _jax()
    return jax.ShapeDtypeStruct(tuple(shape), dtype)


def _ws(nbytes: int):
    _, jnp = _jax()
    return _sds((int(nbytes),), jnp.uint8)


# --------------------------------------------------------------------------------------- attention
def hip_attention(q, k, v, window: int = -1, softcap: float = 0.0):
    """q [B,S,H,D], k/v [B,S,K,D] bf16 -> [B,S,H,D]; causal, GQA, keys i-window..i (window < 0: all)."""
    return _attention(q, k, v, int(window), float(softcap))


@functools.lru_cache(maxsize=None)
def _attention_vjp():
    jax, jnp = _jax()

    @functools.partial(jax.custom_vjp, nondiff_argnums=(3, 4))
    def attention(q, k, v, window, softcap):
        return fwd(q, k, v, window, softcap)[0]

    def fwd(q, k, v, window, softcap):
        B, S, H, D = q.shape
        o, lse = jax.ffi.ffi_call("olmax_attn_fwd", (_sds(q.shape, q.dtype), _sds((B, H, S), jnp.float32)))(
            q, k, v, window=np.int32(window), softcap=np.float32(softcap))
        return o, (q, k, v, o, lse)

    def bwd(window, softcap, res, d_o):
        q, k, v, o, lse = res
        B, S, H, D = q.shape
        L = _lib.load()
        L.olmax_attn_bwd_workspace_bytes.restype = ctypes.c_int64
        L.olmax_attn_bwd_workspace_bytes_aligned.restype = ctypes.c_int64
        # XLA buffers are at least 16-byte aligned and the row strides are heads * D: head_dim 128 takes the
        # MFMA path, whose scratch is delta only (the general query adds two fp32 [B*S, K*D] accumulators)
        nbytes = (L.olmax_attn_bwd_workspace_bytes_aligned(B, S, H) if D == 128
                  else L.olmax_attn_bwd_workspace_bytes(B, S, H, k.shape[2], D))
        dq, dk, dv, _ = jax.ffi.ffi_call(
            "olmax_attn_bwd", (_sds(q.shape, q.dtype), _sds(k.shape, k.dtype), _sds(v.shape, v.dtype), _ws(nbytes)))(
            q, k, v, o, lse, d_o, window=np.int32(window), softcap=np.float32(softcap))
        return dq, dk, dv

    attention.defvjp(fwd, bwd)
    return attention


def _attention(q, k, v, window, softcap):
    return _attention_vjp()(q, k, v, window, softcap)


# --------------------------------------------------------------------------------------- rms_norm
def hip_rms_norm(x, weight, eps: float = 1e-5):
    """olmax.nn.functional.rms_norm for bf16 x [..., d] and weight [d]."""
    return _rms_norm_vjp()(x, weight, float(eps))


@functools.lru_cache(maxsize=None)
def _rms_norm_vjp():
    jax, jnp = _jax()

    @functools.partial(jax.custom_vjp, nondiff_argnums=(2,))
    def rms_norm(x, w, eps):
        return jax.ffi.ffi_call("olmax_rmsnorm_fwd", _sds(x.shape, x.dtype))(x, w, eps=np.float32(eps))

    def fwd(x, w, eps):
        return rms_norm(x, w, eps), (x, w)

    def bwd(eps, res, dy):
        x, w = res
        dx, dw = jax.ffi.ffi_call("olmax_rmsnorm_bwd", (_sds(x.shape, x.dtype), _sds(w.shape, jnp.float32)))(
            x, w, dy, eps=np.float32(eps))
        return dx, dw.astype(w.dtype)

    rms_norm.defvjp(fwd, bwd)
    return rms_norm


# --------------------------------------------------------------------------------------- linear
def hip_linear(x, weight):
    """olmax.nn.functional.linear without bias: x [..., in] @ weight[out, in]^T, bf16."""
    return _linear_vjp()(x, weight)


@functools.lru_cache(maxsize=None)
def _linear_vjp():
    jax, jnp = _jax()

    def gemm(a, b, shape, a_layout, b_layout):
        return jax.ffi.ffi_call("olmax_gemm", _sds(shape, a.dtype))(a, b, a_layout=np.int32(a_layout), b_layout=np.int32(b_layout))

    @jax.custom_vjp
    def linear(x, w):
        return gemm(x.reshape(-1, x.shape[-1]), w, (*x.shape[:-1], w.shape[0]), 0, 0)

    def fwd(x, w):
        return linear(x, w), (x, w)

    def bwd(res, dy):
        x, w = res
        x2, dy2 = x.reshape(-1, x.shape[-1]), dy.reshape(-1, dy.shape[-1])
        dx = gemm(dy2, w, x.shape, 0, 1)       # dx = dy W       (B stored [K=out, N=in])
        dw = gemm(dy2, x2, w.shape, 1, 1)      # dW = dy^T x     (A stored [K=tokens, M=out])
        return dx, dw

    linear.defvjp(fwd, bwd)
    return linear


# --------------------------------------------------------------------------------------- LM head + CE
def hip_lm_head_cross_entropy(h, weight, labels, final_softcap: float = 0.0):
    """mean cross entropy of (h @ weight^T) against int32 labels (ignore_index -100): LMHead.forward
    followed by cross_entropy_loss as in the benchmark's loss_fun
    (src/integration_tests/train_transformer.py:190-206).  Forward and backward are one library call;
    the backward of this op only scales the saved gradients by the incoming cotangent."""
    return _lm_head_vjp()(h, weight, labels, float(final_softcap))


@functools.lru_cache(maxsize=None)
def _lm_head_vjp():
    jax, jnp = _jax()

    # labels is an array (a tracer under jit), so it is a regular argument with no cotangent, not a
    # nondiff_argnums entry (those must be static Python values)
    @functools.partial(jax.custom_vjp, nondiff_argnums=(3,))
    def head(h, w, labels, softcap):
        return fwd(h, w, labels, softcap)[0]

    def fwd(h, w, labels, softcap):
        h2 = h.reshape(-1, h.shape[-1])
        L = _lib.load()
        L.olmax_lmhead_ce_workspace_bytes.restype = ctypes.c_int64
        nbytes = L.olmax_lmhead_ce_workspace_bytes(ctypes.c_int64(h2.shape[0]), ctypes.c_int32(w.shape[0]))
        loss, dh, dw, _ = jax.ffi.ffi_call(
            "olmax_lmhead_ce", (_sds((), jnp.float32), _sds(h2.shape, h.dtype), _sds(w.shape, w.dtype), _ws(nbytes)))(
            h2, w, labels.reshape(-1).astype(jnp.int32), softcap=np.float32(softcap))
        return loss, (dh.reshape(h.shape), dw)

    def bwd(softcap, res, g):
        dh, dw = res
        return (g * dh).astype(dh.dtype), (g * dw).astype(dw.dtype), None

    head.defvjp(fwd, bwd)
    return head


# --------------------------------------------------------------------------------------- cross entropy on logits
_REDUCTIONS = {"mean": 0, "sum": 1, "none": 2}


def hip_fused_cross_entropy_loss(logits, labels, *, ignore_index: int = -100, reduction: str = "mean", softcap: float = 0.0):
    """fused_cross_entropy_loss (src/olmax/nn/functional.py:94-121): (loss, log_normalizer * where) for bf16 or fp32
    logits [..., V]; the log-normaliser comes back shaped [..., 1] like the reference's keepdims output.  Only the
    loss is differentiable here (the reference's z-loss users differentiate the normaliser through XLA)."""
    loss, lse = _cross_entropy_vjp()(logits, labels, int(ignore_index), _REDUCTIONS[reduction], float(softcap))
    return loss, lse.reshape(*logits.shape[:-1], 1)


def hip_cross_entropy_loss(logits, labels, *, ignore_index: int = -100, reduction: str = "mean"):
    """cross_entropy_loss (src/olmax/nn/functional.py:70-91), reduction "mean" | "sum" | "none"."""
    return hip_fused_cross_entropy_loss(logits, labels, ignore_index=ignore_index, reduction=reduction)[0]


@functools.lru_cache(maxsize=None)
def _cross_entropy_vjp():
    jax, jnp = _jax()

    def ws_bytes(T):
        L = _lib.load()
        L.olmax_cross_entropy_workspace_bytes.restype = ctypes.c_int64
        return L.olmax_cross_entropy_workspace_bytes(ctypes.c_int64(T))

    @functools.partial(jax.custom_vjp, nondiff_argnums=(2, 3, 4))
    def ce(logits, labels, ignore_index, reduction, softcap):
        return fwd(logits, labels, ignore_index, reduction, softcap)[0]

    def fwd(logits, labels, ignore_index, reduction, softcap):
        z = logits.reshape(-1, logits.shape[-1])
        T = z.shape[0]
        lab = labels.reshape(-1).astype(jnp.int32)
        loss, lse, _ = jax.ffi.ffi_call(
            "olmax_cross_entropy_fwd", (_sds((T,) if reduction == 2 else (), jnp.float32), _sds((T,), jnp.float32), _ws(ws_bytes(T))))(
            z, lab, reduction=np.int32(reduction), ignore_index=np.int32(ignore_index), softcap=np.float32(softcap))
        if reduction == 2:
            loss = loss.reshape(labels.shape)
        return (loss, lse.reshape(labels.shape)), (logits, lab)

    def bwd(ignore_index, reduction, softcap, res, cts):
        logits, lab = res
        g = cts[0]  # the normaliser's cotangent is not propagated (see hip_fused_cross_entropy_loss)
        z = logits.reshape(-1, logits.shape[-1])
        T = z.shape[0]
        if reduction == 2:
            rows = g.reshape(-1).astype(jnp.float32)
        else:
            n = jnp.sum(lab != ignore_index).astype(jnp.float32) if reduction == 0 else jnp.float32(1.0)
            rows = jnp.broadcast_to(g.astype(jnp.float32) / n, (T,))
        d, _, _ = jax.ffi.ffi_call(
            "olmax_cross_entropy_bwd", (_sds(z.shape, z.dtype), _sds((T,), jnp.float32), _ws(ws_bytes(T))))(
            z, lab, rows, ignore_index=np.int32(ignore_index), softcap=np.float32(softcap))
        return d.reshape(logits.shape), None

    ce.defvjp(fwd, bwd)
    return ce


# --------------------------------------------------------------------------------------- RoPE (+ head-wise QK-norm)
def hip_rope(x, freqs_cos, freqs_sin, norm_weight=None, eps: float = 1e-5):
    """RotaryPositionalEmbedding.forward (src/olmax/nn/rope.py:68-80) for x [B, S, H, D] (head_first=False) with the
    cached tables of get_freqs_cis ([S, D/2] fp32).  With ``norm_weight`` ([D]) the head-wise RMSNorm of
    src/olmax/nn/attention.py:293-296 runs first in the same kernel."""
    _, jnp = _jax()
    w = jnp.ones((x.shape[-1],), x.dtype) if norm_weight is None else norm_weight
    return _rope_vjp()(x, w, freqs_cos, freqs_sin, norm_weight is not None, float(eps))


@functools.lru_cache(maxsize=None)
def _rope_vjp():
    jax, jnp = _jax()

    @functools.partial(jax.custom_vjp, nondiff_argnums=(4, 5))
    def rope(x, w, cos, sin, use_norm, eps):
        return jax.ffi.ffi_call("olmax_qk_rope_fwd", _sds(x.shape, x.dtype))(
            x, w, cos.astype(jnp.float32), sin.astype(jnp.float32), use_norm=np.int32(use_norm), eps=np.float32(eps))

    def fwd(x, w, cos, sin, use_norm, eps):
        return rope(x, w, cos, sin, use_norm, eps), (x, w, cos, sin)

    def bwd(use_norm, eps, res, dy):
        x, w, cos, sin = res
        dx, dw = jax.ffi.ffi_call("olmax_qk_rope_bwd", (_sds(x.shape, x.dtype), _sds(w.shape, jnp.float32)))(
            dy, x, w, cos.astype(jnp.float32), sin.astype(jnp.float32), use_norm=np.int32(use_norm), eps=np.float32(eps))
        return dx, dw.astype(w.dtype), jnp.zeros_like(cos), jnp.zeros_like(sin)

    rope.defvjp(fwd, bwd)
    return rope


# --------------------------------------------------------------------------------------- gated MLP input half
_ACTS = {"silu": 0, "gelu": 1}


def hip_gated_mlp_in(x, gate_weight, up_weight, activation: str = "silu"):
    """act(gate_proj(x)) * up_proj(x) of GatedMLP.forward (src/olmax/nn/mlp.py:69-73) as ONE GEMM over
    [Wgate; Wup] with the activation in its epilogue; the down projection stays ``hip_linear``.  (The Equinox
    module owns two Linear layers, so the two weights are concatenated per call; a module that stores them
    adjacent, as the flat layout of ``HipTrainStep`` does, skips that copy.)"""
    return _gated_vjp()(x, gate_weight, up_weight, _ACTS[activation])


@functools.lru_cache(maxsize=None)
def _gated_vjp():
    jax, jnp = _jax()
    linear = _linear_vjp()

    @functools.partial(jax.custom_vjp, nondiff_argnums=(3,))
    def gated(x, wg, wu, act):
        return fwd(x, wg, wu, act)[0]

    def fwd(x, wg, wu, act):
        F = wg.shape[0]
        w = jnp.concatenate([wg, wu], axis=0)
        out, gu = jax.ffi.ffi_call("olmax_gemm_glu", (_sds((*x.shape[:-1], F), x.dtype), _sds((*x.shape[:-1], 2 * F), x.dtype)))(
            x, w, act=np.int32(act))
        return out, (x, w, gu)

    def bwd(act, res, dh):
        x, w, gu = res
        F = w.shape[0] // 2
        dgu = jax.ffi.ffi_call("olmax_glu_bwd", _sds(gu.shape, gu.dtype))(gu, dh, act=np.int32(act))
        x2, dgu2 = x.reshape(-1, x.shape[-1]), dgu.reshape(-1, 2 * F)
        dx = jax.ffi.ffi_call("olmax_gemm", _sds(x.shape, x.dtype))(dgu2, w, a_layout=np.int32(0), b_layout=np.int32(1))
        dw = jax.ffi.ffi_call("olmax_gemm", _sds(w.shape, w.dtype))(dgu2, x2, a_layout=np.int32(1), b_layout=np.int32(1))
        return dx, dw[:F], dw[F:]

    gated.defvjp(fwd, bwd)
    return gated


# --------------------------------------------------------------------------------------- embedding
def hip_embedding(weight, ids):
    """Embedding.forward (src/olmax/nn/embedding.py:30-32): rows of weight [V, d] (bf16) for integer ids of any
    shape; the backward is the fp32 scatter-add, cast back to the weight's dtype."""
    return _embedding_vjp()(weight, ids)


@functools.lru_cache(maxsize=None)
def _embedding_vjp():
    jax, jnp = _jax()

    @jax.custom_vjp
    def embed(w, ids):
        return jax.ffi.ffi_call("olmax_embed_fwd", _sds((*ids.shape, w.shape[1]), w.dtype))(ids.astype(jnp.int32), w)

    def fwd(w, ids):
        return embed(w, ids), (w, ids)

    def bwd(res, dh):
        w, ids = res
        dw = jax.ffi.ffi_call("olmax_embed_bwd", _sds(w.shape, jnp.float32))(ids.astype(jnp.int32), dh)
        return dw.astype(w.dtype), None

    embed.defvjp(fwd, bwd)
    return embed


# --------------------------------------------------------------------------------------- optimizer
def _hyper(jnp, lr, count, b1, b2):
    """fp32 [3] = {lr, 1 - b1^t, 1 - b2^t} for the 1-based step t = count + 1, on the device."""
    t = (count + 1).astype(jnp.float32)
    return jnp.stack([jnp.asarray(lr, jnp.float32), 1.0 - jnp.float32(b1) ** t, 1.0 - jnp.float32(b2) ** t])


def hip_adamw(learning_rate, b1=0.9, b2=0.999, eps=1e-8, weight_decay=1e-4, mask=None):
    """optax.GradientTransformation whose update runs the fused AdamW per leaf and returns
    ``p_new - p`` so that ``eqx.apply_updates`` (src/olmax/train/trainer.py:752) stays as it is.
    State: (count, mu, nu) like optax.adamw; the learning rate is read at the pre-increment count.
    lr and the bias corrections travel as a 3-element device buffer, so the update is traceable
    under jit without a host read-back.  ``mask``: pytree of bools, False = no weight decay
    (AdamWConfig.build's weight_decay_mask, src/olmax/optim/config.py:136-148)."""
    jax, jnp = _jax()
    import optax

    def init(params):
        z = jax.tree.map(lambda p: jnp.zeros_like(p, dtype=jnp.float32), params)
        return (jnp.zeros([], jnp.int32), z, jax.tree.map(jnp.copy, z))

    def update(grads, state, params):
        count, mu, nu = state
        lr = learning_rate(count) if callable(learning_rate) else learning_rate
        hyper = _hyper(jnp, lr, count, b1, b2)
        decays = jax.tree.map(lambda _: True, params) if mask is None else mask

        def leaf(p, g, m, v, d):
            p2, m2, v2 = jax.ffi.ffi_call(
                "olmax_adamw", (_sds(p.shape, p.dtype), _sds(m.shape, m.dtype), _sds(v.shape, v.dtype)),
                input_output_aliases={0: 0, 2: 1, 3: 2})(
                jnp.copy(p), g, m, v, hyper, b1=np.float32(b1), b2=np.float32(b2), eps=np.float32(eps),
                wd=np.float32(weight_decay if d else 0.0))
            return p2 - p, m2, v2

        out = jax.tree.map(leaf, params, grads, mu, nu, decays)
        pick = lambda i: jax.tree.map(lambda t: t[i], out, is_leaf=lambda t: isinstance(t, tuple))
        return pick(0), (count + 1, pick(1), pick(2))

    return optax.GradientTransformation(init, update)


# --------------------------------------------------------------------------------------- whole step
class HipTrainStep:
    """process_microbatch as one custom call.

    ``pack(model)`` copies the Equinox model's leaves ONCE into the flat fp32 master buffer (layout
    of ``olmax_amd.layout.leaf_table``: the reference's leaf names at fixed offsets, q|k|v and gate|up
    adjacent) and builds m, v (zeros) and the bf16 working copy; ``__call__(state, ids, labels, count)``
    is the jitted, donating equivalent of the reference's process_microbatch: the four state buffers
    go in and come back aliased, the loss comes back as a device scalar; ``count`` (device int32, the
    number of optimizer steps taken so far) and the schedule stay on the device.  ``unpack(state)``
    gives the leaves back by name (checkpointing, evaluation with the reference's own modules)."""

    def __init__(self, config, *, batch_size: int, sequence_length: int, learning_rate=1e-4, b1=0.9, b2=0.999, eps=1e-8, weight_decay=1e-4,
                 no_decay_modules: Optional[Sequence[str]] = None, max_grad_norm: Optional[float] = None,
                 overlap_optimizer: bool = True):
        import fnmatch

        from . import layout

        jax, jnp = _jax()
        register()
        self.config, self.B, self.S = config, batch_size, sequence_length
        self.table = layout.leaf_table(config, batch_size, sequence_length)
        self.n = layout.num_params(config)
        c = config.c_config(batch_size, sequence_length)
        L = _lib.load()
        L.olmax_model_workspace_bytes.restype = ctypes.c_int64
        L.olmax_model_grad_f32_elems.restype = ctypes.c_int64
        self.ws_bytes = int(L.olmax_model_workspace_bytes(ctypes.byref(c)))
        self.nf = int(L.olmax_model_grad_f32_elems(ctypes.byref(c)))
        pats = list(no_decay_modules or [])
        decay = [0 if any(fnmatch.fnmatch(l.name, p) for p in pats) else 1 for l in self.table] if pats else []
        thetas = config.thetas()
        uniq = sorted(set(thetas))
        ints = [getattr(c, f) for f, _ in c._fields_[:14]]
        # attributes of the custom call are host values (numpy), fixed when the step is traced
        attrs = dict(config=np.asarray(ints, np.int32), eps=np.float32(c.eps), attn_softcap=np.float32(c.attn_softcap),
                     final_softcap=np.float32(c.final_softcap), windows=np.asarray(config.windows(), np.int32),
                     table_index=np.asarray([uniq.index(t) for t in thetas], np.int32),
                     leaf_decay=np.asarray(decay, np.int32), b1=np.float32(b1), b2=np.float32(b2),
                     adam_eps=np.float32(eps), wd=np.float32(weight_decay), max_grad_norm=np.float32(max_grad_norm or 0.0),
                     overlap=np.int32(int(overlap_optimizer and not max_grad_norm)))
        # cos/sin tables, formed in fp32 as src/olmax/nn/rope.py:127-133 does
        half = jnp.arange(0.0, config.head_dim, 2) / config.head_dim
        ang = jnp.stack([jnp.outer(jnp.arange(float(sequence_length)), 1.0 / (jnp.float32(t) ** half)) for t in uniq])
        self.cos, self.sin = jnp.cos(ang), jnp.sin(ang)
        n, nf, T = self.n, self.nf, batch_size * sequence_length

        def step_fn(master, m, v, params, ids, labels, cos, sin, count):
            lr = learning_rate(count) if callable(learning_rate) else learning_rate  # read at the pre-increment count
            hyper = _hyper(jnp, lr, count, b1, b2)
            outs = jax.ffi.ffi_call(
                "olmax_train_step",
                (_sds((n,), jnp.float32), _sds((n,), jnp.float32), _sds((n,), jnp.float32), _sds((n,), jnp.bfloat16),
                 _sds((), jnp.float32), _sds((n,), jnp.bfloat16), _sds((nf,), jnp.float32), _ws(self.ws_bytes),
                 _sds((2,), jnp.float32)),
                input_output_aliases={0: 0, 1: 1, 2: 2, 3: 3}, has_side_effect=True)(
                master, m, v, params, ids.reshape(T).astype(jnp.int32), labels.reshape(T).astype(jnp.int32), cos, sin,
                hyper, **attrs)
            return outs[:4], outs[4], outs[8]

        self._step = jax.jit(step_fn, donate_argnums=(0, 1, 2, 3))

    def pack(self, model):
        """Equinox model (fp32 leaves under the reference's names) -> (master, m, v, params_bf16)."""
        import equinox as eqx

        jax, jnp = _jax()
        named = {}
        for path, leaf in jax.tree_util.tree_flatten_with_path(eqx.filter(model, eqx.is_array))[0]:
            name = ".".join(str(getattr(k, "name", getattr(k, "idx", k))) for k in path)
            named[name] = leaf
        master = jnp.concatenate([named[l.name].astype(jnp.float32).reshape(-1) for l in self.table])
        assert master.shape == (self.n,)  # the leaves tile the flat buffer in layout order, without gaps
        return master, jnp.zeros_like(master), jnp.zeros_like(master), master.astype(jnp.bfloat16)

    def unpack(self, state):
        master = state[0]
        out = {}
        for l in self.table:
            k = 1
            for s in l.shape:
                k *= s
            out[l.name] = master[l.offset: l.offset + k].reshape(l.shape)
        return out

    def __call__(self, state, input_ids, labels, count):
        """-> (new state, loss, [clip factor, grad norm]); ``count``: optimizer steps taken so far."""
        new_state, loss, norm = self._step(*state, input_ids, labels, self.cos, self.sin, count)
        return tuple(new_state), loss, norm
