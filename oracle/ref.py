"""CPU oracle: an independent restatement of OLMax's transformer training hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this module; it is
used by ``tests/``, by ``__graft_entry__.smoke()`` as the checker and by ``bench.py`` for
its ``cpu_baseline`` leg.

The reference (epwalsh/OLMax) is pure JAX/Equinox and cannot be imported where this
runs, and its backward pass is never written down (it comes from
``eqx.filter_value_and_grad``, src/olmax/train/trainer.py:734).  Every function here
therefore restates a reference forward from the cited file:line in plain torch-CPU
arithmetic and gives a hand-derived backward.  ``tests/test_oracle.py`` pins each one
with something that does not share its formula: backward formulas against
``torch.autograd``, forwards against closed forms, textbook routines
(``torch.nn.functional``, ``scipy``, ``torch.optim.AdamW``), hand-computed examples and
invariants; the three block orderings against a block rebuilt from torch's own routines;
``train_step`` / ``train_batch`` (micro-batch running mean, global-norm clip, masked
decay) against autograd of the mean loss plus a hand-computed clip factor plus
``torch.optim.AdamW``; the fp32 RoPE table against the closed form by an ulp bound.

Parity status: every function below has such a check.  What no check here can reach
(the reference's tests hold no numeric vectors for these ops, and JAX / optax cannot be
imported): the attention window off-by-one, the tanh-GELU default, optax's epsilon
placement and MultiSteps averaging follow upstream documentation ("parity unpinned" by
reference fixtures); soft-caps, tied embeddings and per-layer windows have no reference
implementation at all.

Rounding model: ``rt`` ("round to") is applied exactly where the reference's bf16 compute
path rounds (every op output is an array of the compute dtype).  With ``rt=None`` the
arithmetic is done in whatever dtype the inputs carry (fp64 for exact checks).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Callable, Optional

import torch

Tensor = torch.Tensor


def bf16_round(x: Tensor) -> Tensor:
    """Round-to-nearest-even to bf16, keep the container dtype."""
    return x.to(torch.bfloat16).to(x.dtype)


def _id(x: Tensor) -> Tensor:
    return x


# --------------------------------------------------------------------------- RMSNorm
def rms_norm_fwd(x: Tensor, w: Optional[Tensor], eps: float, rt=_id) -> Tensor:
    """src/olmax/nn/functional.py:51-67 — y = w * (rsqrt(mean(x^2) + eps) * x), in fp32+."""
    r = torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)
    y = r * x
    if w is not None:
        y = w * y
    return rt(y)


def rms_norm_bwd(x: Tensor, w: Optional[Tensor], dy: Tensor, eps: float, rt=_id):
    """Hand-derived transpose of rms_norm_fwd.

    g = w*dy;  dx = r*g - x * r^3 * mean(x*g);  dw = sum_rows dy * x * r.
    """
    r = torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)
    g = dy if w is None else w * dy
    dx = r * g - x * (r ** 3) * (x * g).mean(-1, keepdim=True)
    dw = None
    if w is not None:
        dw = (dy * x * r).reshape(-1, x.shape[-1]).sum(0)
        dw = rt(dw)
    return rt(dx), dw


# --------------------------------------------------------------------------- RoPE
def rope_tables(seq_len: int, head_dim: int, theta: float, dtype=torch.float32):
    """src/olmax/nn/rope.py:118-145 — cos/sin of outer(arange(S), theta^(-2i/D)), [S, D/2].

    The reference forms `freqs`, `t` and their outer product in its default float type
    (fp32: `jnp.arange(0.0, head_dim, 2)`, `jnp.arange(float(end))`, rope.py:127-130) and only
    the cos/sin results take `dtype`; every intermediate below is therefore an array of
    `dtype` itself (fp32 by default; fp64 gives the exact closed form for checks)."""
    exponent = torch.arange(0.0, head_dim, 2, dtype=dtype) / head_dim
    freqs = 1.0 / torch.pow(torch.tensor(theta, dtype=dtype), exponent)
    t = torch.arange(float(seq_len), dtype=dtype)
    ang = torch.outer(t, freqs)
    return torch.cos(ang), torch.sin(ang)


def rope_fwd(x: Tensor, cos: Tensor, sin: Tensor, rt=_id) -> Tensor:
    """src/olmax/nn/rope.py:62-65,99-115 — x*cos + rotate_half(x)*sin, half-split pairing.

    x: [B, S, H, D]; cos/sin: [S, D/2].
    """
    d2 = x.shape[-1] // 2
    c = cos.to(x.dtype)[None, :, None, :]
    s = sin.to(x.dtype)[None, :, None, :]
    x1, x2 = x[..., :d2], x[..., d2:]
    return rt(torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], -1))


def rope_bwd(dy: Tensor, cos: Tensor, sin: Tensor, rt=_id) -> Tensor:
    """Transpose of rope_fwd: rotation by the negative angle."""
    d2 = dy.shape[-1] // 2
    c = cos.to(dy.dtype)[None, :, None, :]
    s = sin.to(dy.dtype)[None, :, None, :]
    d1, dd2 = dy[..., :d2], dy[..., d2:]
    return rt(torch.cat([d1 * c + dd2 * s, dd2 * c - d1 * s], -1))


# --------------------------------------------------------------------------- Linear
def linear_fwd(x: Tensor, w: Tensor, rt=_id) -> Tensor:
    """src/olmax/nn/functional.py:14-27 — y = x W^T with W stored [out, in]."""
    return rt(x @ w.transpose(-1, -2))


def linear_bwd(x: Tensor, w: Tensor, dy: Tensor, rt=_id):
    """dx = dy W ; dW = dy^T x (summed over all leading dims)."""
    dx = rt(dy @ w)
    dw = rt(dy.reshape(-1, dy.shape[-1]).t() @ x.reshape(-1, x.shape[-1]))
    return dx, dw


# --------------------------------------------------------------------------- gated MLP activation
_GELU_C = math.sqrt(2.0 / math.pi)


def act_fwd(g: Tensor, kind: str) -> Tensor:
    """silu: jax.nn.silu (src/olmax/nn/mlp.py:24); gelu: jax.nn.gelu default = tanh
    approximation (src/olmax/nn/transformer/layer.py:133)."""
    if kind == "silu":
        return g * torch.sigmoid(g)
    if kind == "gelu":
        return 0.5 * g * (1.0 + torch.tanh(_GELU_C * (g + 0.044715 * g ** 3)))
    raise ValueError(kind)


def act_grad(g: Tensor, kind: str) -> Tensor:
    if kind == "silu":
        s = torch.sigmoid(g)
        return s * (1.0 + g * (1.0 - s))
    if kind == "gelu":
        t = torch.tanh(_GELU_C * (g + 0.044715 * g ** 3))
        return 0.5 * (1.0 + t) + 0.5 * g * (1.0 - t * t) * _GELU_C * (1.0 + 3 * 0.044715 * g * g)
    raise ValueError(kind)


def glu_fwd(gate: Tensor, up: Tensor, kind: str, rt=_id) -> Tensor:
    """src/olmax/nn/mlp.py:69-73 — act(gate(x)) * up(x).  The reference rounds act(gate) to
    the compute dtype before the product (two separate XLA ops on bf16 arrays)."""
    return rt(rt(act_fwd(gate, kind)) * up)


def glu_bwd(gate: Tensor, up: Tensor, dh: Tensor, kind: str, rt=_id):
    dgate = rt(dh * up * act_grad(gate, kind))
    dup = rt(dh * act_fwd(gate, kind))
    return dgate, dup


# --------------------------------------------------------------------------- attention
def attention_mask(S: int, window: Optional[int]) -> Tensor:
    """Causal mask j <= i, optionally j >= i - window (JAX local_window_size=(w, w) combined
    with is_causal=True, called at src/olmax/nn/attention.py:96-103): w + 1 visible keys."""
    i = torch.arange(S)[:, None]
    j = torch.arange(S)[None, :]
    m = j <= i
    if window is not None:
        m = m & (j >= i - window)
    return m


def attention_fwd(q: Tensor, k: Tensor, v: Tensor, *, window: Optional[int] = None,
                  softcap: float = 0.0, rt=_id):
    """Brute-force causal GQA attention, BSHD (src/olmax/nn/attention.py:52-109).

    q: [B,S,H,D], k/v: [B,S,K,D].  Query head h reads kv head h // (H/K).
    Returns (o [B,S,H,D], lse [B,H,S]).  P is rounded (rt) before the PV product, as the
    upstream XLA path casts probabilities to V's dtype.
    """
    B, S, H, D = q.shape
    K = k.shape[2]
    rep = H // K
    scale = 1.0 / math.sqrt(D)
    kk = k.repeat_interleave(rep, dim=2)
    vv = v.repeat_interleave(rep, dim=2)
    s = torch.einsum("bihd,bjhd->bhij", q, kk) * scale
    if softcap and softcap > 0:
        s = softcap * torch.tanh(s / softcap)
    mask = attention_mask(S, window)
    s = s.masked_fill(~mask, float("-inf"))
    lse = torch.logsumexp(s, -1)
    p = torch.exp(s - lse[..., None])
    o = torch.einsum("bhij,bjhd->bihd", rt(p), vv)
    return rt(o), lse


def attention_bwd(q, k, v, o, lse, do, *, window=None, softcap: float = 0.0, rt=_id):
    """Hand-derived: dV = P^T dO; dP = dO V^T; dS = P*(dP - rowsum(dO*O));
    soft-cap chain factor (1 - tanh^2); dQ = dS K * scale; dK = dS^T Q * scale.
    kv-head grads are summed over the H/K query heads that share them."""
    B, S, H, D = q.shape
    K = k.shape[2]
    rep = H // K
    scale = 1.0 / math.sqrt(D)
    kk = k.repeat_interleave(rep, dim=2)
    vv = v.repeat_interleave(rep, dim=2)
    s_raw = torch.einsum("bihd,bjhd->bhij", q, kk) * scale
    if softcap and softcap > 0:
        t = torch.tanh(s_raw / softcap)
        s = softcap * t
    else:
        t = None
        s = s_raw
    mask = attention_mask(S, window)
    p = torch.exp(s - lse[..., None]).masked_fill(~mask, 0.0)
    dv_full = torch.einsum("bhij,bihd->bjhd", rt(p), do)
    dp = torch.einsum("bihd,bjhd->bhij", do, vv)
    delta = (do * o).sum(-1).permute(0, 2, 1)  # [B,H,S]
    ds = p * (dp - delta[..., None])
    if t is not None:
        ds = ds * (1.0 - t * t)
    ds = rt(ds)
    dq = torch.einsum("bhij,bjhd->bihd", ds, kk) * scale
    dk_full = torch.einsum("bhij,bihd->bjhd", ds, q) * scale
    dk = dk_full.reshape(B, S, K, rep, D).sum(3)
    dv = dv_full.reshape(B, S, K, rep, D).sum(3)
    return rt(dq), rt(dk), rt(dv)


# --------------------------------------------------------------------------- cross entropy
def cross_entropy_fwd(logits: Tensor, labels: Tensor, ignore_index: int = -100,
                      softcap: float = 0.0, reduction: str = "mean"):
    """src/olmax/nn/functional.py:70-91; reduction "mean" (default), "sum" or "none" (:84-91).

    Quirks kept: a label outside [0, V) that is not ignore_index has an all-zero one-hot, so
    its loss is 0 but it still counts in the mean's denominator; ignore_index rows count in
    neither.  Returns (loss, lse[T], n_counted).
    """
    V = logits.shape[-1]
    z = logits
    if softcap and softcap > 0:
        z = softcap * torch.tanh(z / softcap)
    where = labels != ignore_index
    inrange = (labels >= 0) & (labels < V)
    lse = torch.logsumexp(z, -1)
    tgt = torch.gather(z, -1, labels.clamp(0, V - 1)[..., None].long())[..., 0]
    per = torch.where(where & inrange, lse - tgt, torch.zeros_like(lse))
    n = where.sum()
    if reduction == "mean":
        loss = per.sum() / n
    elif reduction == "sum":
        loss = per.sum()
    elif reduction == "none":
        loss = per
    else:
        raise ValueError(reduction)
    return loss, lse, n


def cross_entropy_bwd(logits: Tensor, labels: Tensor, ignore_index: int = -100,
                      softcap: float = 0.0, dloss=1.0, reduction: str = "mean") -> Tensor:
    """dlogits_i = (softmax_i - onehot_i) * dloss / n for counted in-range rows, 0 otherwise
    ("sum": no division by n; "none": dloss is the per-row cotangent [T])."""
    V = logits.shape[-1]
    z = logits
    t = None
    if softcap and softcap > 0:
        t = torch.tanh(z / softcap)
        z = softcap * t
    where = labels != ignore_index
    inrange = (labels >= 0) & (labels < V)
    n = where.sum()
    p = torch.softmax(z, -1)
    oh = torch.nn.functional.one_hot(labels.clamp(0, V - 1).long(), V).to(z.dtype)
    if reduction == "mean":
        scale = dloss / n
    elif reduction == "sum":
        scale = dloss
    else:
        scale = torch.as_tensor(dloss, dtype=z.dtype).reshape(-1, 1) * torch.ones(z.shape[0], 1, dtype=z.dtype)
    d = (p - oh) * (where & inrange)[..., None].to(z.dtype) * scale
    if t is not None:
        d = d * (1.0 - t * t)
    return d


def lm_head_ce(h: Tensor, w: Tensor, labels: Tensor, *, softcap: float = 0.0, rt=_id,
               ignore_index: int = -100):
    """LMHead (src/olmax/nn/lm_head.py:59-61: logits = (h W^T) in compute dtype, widened to
    fp32) followed by cross_entropy_loss.  Returns loss, dh, dW."""
    logits = rt(h @ w.t())
    loss, lse, n = cross_entropy_fwd(logits, labels, ignore_index, softcap)
    dlogits = rt(cross_entropy_bwd(logits, labels, ignore_index, softcap))
    dh = rt(dlogits @ w)
    dw = rt(dlogits.reshape(-1, dlogits.shape[-1]).t() @ h.reshape(-1, h.shape[-1]))
    return loss, dh, dw


# --------------------------------------------------------------------------- embedding
def embed_fwd(ids: Tensor, w: Tensor) -> Tensor:
    """src/olmax/nn/embedding.py:30-32 — row gather."""
    return w[ids.long()]


def embed_bwd(ids: Tensor, dh: Tensor, vocab: int) -> Tensor:
    """Scatter-add; duplicate ids sum."""
    dw = torch.zeros(vocab, dh.shape[-1], dtype=dh.dtype)
    dw.index_add_(0, ids.reshape(-1).long(), dh.reshape(-1, dh.shape[-1]))
    return dw


# --------------------------------------------------------------------------- AdamW
def adamw_step(p, g, m, v, *, step: int, lr: float, b1: float = 0.9, b2: float = 0.999,
               eps: float = 1e-8, wd: float = 1e-4):
    """optax.adamw as configured at src/olmax/optim/config.py:136-156 and applied at
    src/olmax/train/trainer.py:745-752.  `step` is the 1-based count after increment.

    m = b1 m + (1-b1) g; v = b2 v + (1-b2) g^2; mhat = m/(1-b1^t); vhat = v/(1-b2^t);
    p <- p - lr * (mhat / (sqrt(vhat) + eps) + wd * p)
    """
    m = b1 * m + (1 - b1) * g
    v = b2 * v + (1 - b2) * g * g
    mh = m / (1 - b1 ** step)
    vh = v / (1 - b2 ** step)
    p = p - lr * (mh / (torch.sqrt(vh) + eps) + wd * p)
    return p, m, v


# --------------------------------------------------------------------------- LR schedule
def warmup_cosine_lr(step: int, *, warmup_steps: int, decay_steps: int, peak: float,
                     init: float, end: float) -> float:
    """src/olmax/optim/config.py:35-52 → optax.warmup_cosine_decay_schedule with
    decay_steps = warmup_steps + decay_steps (total): linear init→peak over warmup, then
    cosine peak→end over the remaining steps."""
    if step < warmup_steps:
        return init + (peak - init) * step / max(1, warmup_steps)
    t = min(max(step - warmup_steps, 0), decay_steps)
    cos = 0.5 * (1 + math.cos(math.pi * t / max(1, decay_steps)))
    return end + (peak - end) * cos


def wsd_lr(step: int, *, warmup_steps: int, stable_steps: int, decay_steps: int, peak: float,
           init: float = 0.0, end: float = 0.0) -> float:
    """Warmup-stable-decay (linear) schedule, src/olmax/optim/config.py:55-80; pinned by the
    reference's known-answer test src/test/optim/config_test.py:22-33."""
    if step < warmup_steps:
        return init + (peak - init) * step / warmup_steps
    if step < warmup_steps + stable_steps:
        return peak
    t = min(step - warmup_steps - stable_steps, decay_steps)
    return peak + (end - peak) * t / decay_steps


# --------------------------------------------------------------------------- synthetic data
def sequential_tokens(offsets: Tensor, seq_len: int, vocab: int):
    """src/olmax/data/utils.py:12-33 — inputs = (arange(S) + offset) mod V, targets = inputs+1
    (so a target equals V whenever the input is V-1)."""
    ar = torch.arange(seq_len, dtype=torch.int64)[None, :]
    inputs = (ar + offsets[:, None].to(torch.int64)) % vocab
    return inputs.to(torch.int32), (inputs + 1).to(torch.int32)


# --------------------------------------------------------------------------- model
@dataclass
class ModelConfig:
    vocab: int
    d_model: int
    n_layers: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    hidden: int
    layer_type: str = "pre"        # "pre" | "reordered" | "gemma"
    act: str = "silu"              # "silu" | "gelu"
    qk_norm: bool = False          # QK-norm on (src/olmax/nn/attention.py:239-253)
    qk_norm_headwise: bool = True  # True: weight [D] per head (:293-296); False: full width (:281-284)
    eps: float = 1e-6
    rope_theta: float = 10000.0
    rope_theta_layers: Optional[list] = None   # per-layer override
    windows: Optional[list] = None             # per-layer window (None = global)
    attn_softcap: float = 0.0
    final_softcap: float = 0.0
    tied: bool = False

    def theta(self, l: int) -> float:
        return self.rope_theta if self.rope_theta_layers is None else self.rope_theta_layers[l]

    def window(self, l: int):
        return None if self.windows is None else self.windows[l]


def init_params(cfg: ModelConfig, seed: int = 0, std: float = 0.02, dtype=torch.float32) -> dict:
    """Deterministic N(0, std) weights, ones for norm weights.  Leaf names follow the
    reference's pytree paths (src/olmax/nn/transformer/layer.py:21-24,120-121;
    src/olmax/nn/attention.py:113-120; src/olmax/nn/mlp.py:14-16)."""
    g = torch.Generator().manual_seed(seed)
    d, D, H, K, F = cfg.d_model, cfg.head_dim, cfg.n_heads, cfg.n_kv_heads, cfg.hidden

    def n(*shape):
        return (torch.randn(*shape, generator=g, dtype=torch.float32) * std).to(dtype)

    p = {"embedding.weight": n(cfg.vocab, d)}
    for l in range(cfg.n_layers):
        pre = f"layers.{l}."
        p[pre + "attention.q_proj.weight"] = n(H * D, d)
        p[pre + "attention.k_proj.weight"] = n(K * D, d)
        p[pre + "attention.v_proj.weight"] = n(K * D, d)
        p[pre + "attention.o_proj.weight"] = n(d, H * D)
        if cfg.qk_norm:
            # full width: the reference sizes both weights n_heads*head_dim (attention.py:239-253),
            # which only fits k when n_kv_heads == n_heads; k's own width is used here
            p[pre + "attention.q_norm.weight"] = torch.ones(D if cfg.qk_norm_headwise else H * D, dtype=dtype)
            p[pre + "attention.k_norm.weight"] = torch.ones(D if cfg.qk_norm_headwise else K * D, dtype=dtype)
        p[pre + "mlp.gate_proj.weight"] = n(F, d)
        p[pre + "mlp.up_proj.weight"] = n(F, d)
        p[pre + "mlp.down_proj.weight"] = n(d, F)
        p[pre + "attention_norm.weight"] = torch.ones(d, dtype=dtype)
        p[pre + "mlp_norm.weight"] = torch.ones(d, dtype=dtype)
        if cfg.layer_type == "gemma":
            p[pre + "attention_input_norm.weight"] = torch.ones(d, dtype=dtype)
            p[pre + "mlp_input_norm.weight"] = torch.ones(d, dtype=dtype)
    p["norm.weight"] = torch.ones(d, dtype=dtype)
    if not cfg.tied:
        p["lm_head.proj.weight"] = n(cfg.vocab, d)
    return p


class _Tape:
    """Saved forward values of one block (what autodiff would keep)."""

    def __init__(self):
        self.t = {}


def _attn_fwd(cfg, P, pre, l, x, tape, rt):
    B, S, d = x.shape
    H, K, D = cfg.n_heads, cfg.n_kv_heads, cfg.head_dim
    q = linear_fwd(x, P[pre + "attention.q_proj.weight"], rt)
    k = linear_fwd(x, P[pre + "attention.k_proj.weight"], rt)
    v = linear_fwd(x, P[pre + "attention.v_proj.weight"], rt).reshape(B, S, K, D)
    if cfg.qk_norm and cfg.qk_norm_headwise:  # after the reshape (src/olmax/nn/attention.py:293-296)
        q, k = q.reshape(B, S, H, D), k.reshape(B, S, K, D)
    tape["q0"], tape["k0"] = q, k
    if cfg.qk_norm:  # full width: before the reshape (src/olmax/nn/attention.py:281-284)
        q = rms_norm_fwd(q, P[pre + "attention.q_norm.weight"], cfg.eps, rt)
        k = rms_norm_fwd(k, P[pre + "attention.k_norm.weight"], cfg.eps, rt)
    q, k = q.reshape(B, S, H, D), k.reshape(B, S, K, D)
    cos, sin = rope_tables(S, D, cfg.theta(l))
    q = rope_fwd(q, cos, sin, rt)
    k = rope_fwd(k, cos, sin, rt)
    o, lse = attention_fwd(q, k, v, window=cfg.window(l), softcap=cfg.attn_softcap, rt=rt)
    tape.update(q=q, k=k, v=v, o=o, lse=lse, cos=cos, sin=sin, attn_in=x)
    o2 = o.reshape(B, S, H * D)
    return linear_fwd(o2, P[pre + "attention.o_proj.weight"], rt)


def _attn_bwd(cfg, P, pre, l, dy, tape, G, rt):
    B, S, d = dy.shape
    H, K, D = cfg.n_heads, cfg.n_kv_heads, cfg.head_dim
    o2 = tape["o"].reshape(B, S, H * D)
    do, G[pre + "attention.o_proj.weight"] = linear_bwd(o2, P[pre + "attention.o_proj.weight"], dy, rt)
    dq, dk, dv = attention_bwd(tape["q"], tape["k"], tape["v"], tape["o"], tape["lse"],
                               do.reshape(B, S, H, D), window=cfg.window(l),
                               softcap=cfg.attn_softcap, rt=rt)
    dq = rope_bwd(dq, tape["cos"], tape["sin"], rt)
    dk = rope_bwd(dk, tape["cos"], tape["sin"], rt)
    if cfg.qk_norm:
        dq, G[pre + "attention.q_norm.weight"] = rms_norm_bwd(tape["q0"], P[pre + "attention.q_norm.weight"], dq.reshape(tape["q0"].shape), cfg.eps, rt)
        dk, G[pre + "attention.k_norm.weight"] = rms_norm_bwd(tape["k0"], P[pre + "attention.k_norm.weight"], dk.reshape(tape["k0"].shape), cfg.eps, rt)
    x = tape["attn_in"]
    dxq, G[pre + "attention.q_proj.weight"] = linear_bwd(x, P[pre + "attention.q_proj.weight"], dq.reshape(B, S, H * D), rt)
    dxk, G[pre + "attention.k_proj.weight"] = linear_bwd(x, P[pre + "attention.k_proj.weight"], dk.reshape(B, S, K * D), rt)
    dxv, G[pre + "attention.v_proj.weight"] = linear_bwd(x, P[pre + "attention.v_proj.weight"], dv.reshape(B, S, K * D), rt)
    return rt(dxq + dxk + dxv)


def _mlp_fwd(cfg, P, pre, x, tape, rt):
    g = linear_fwd(x, P[pre + "mlp.gate_proj.weight"], rt)
    u = linear_fwd(x, P[pre + "mlp.up_proj.weight"], rt)
    a = glu_fwd(g, u, cfg.act, rt)
    tape.update(mlp_in=x, gate=g, up=u, act=a)
    return linear_fwd(a, P[pre + "mlp.down_proj.weight"], rt)


def _mlp_bwd(cfg, P, pre, dy, tape, G, rt):
    da, G[pre + "mlp.down_proj.weight"] = linear_bwd(tape["act"], P[pre + "mlp.down_proj.weight"], dy, rt)
    dg, du = glu_bwd(tape["gate"], tape["up"], da, cfg.act, rt)
    dxg, G[pre + "mlp.gate_proj.weight"] = linear_bwd(tape["mlp_in"], P[pre + "mlp.gate_proj.weight"], dg, rt)
    dxu, G[pre + "mlp.up_proj.weight"] = linear_bwd(tape["mlp_in"], P[pre + "mlp.up_proj.weight"], du, rt)
    return rt(dxg + dxu)


def block_fwd(cfg: ModelConfig, P: dict, l: int, x: Tensor, rt=_id):
    """The three residual orderings of src/olmax/nn/transformer/layer.py:80-94 (pre),
    :102-116 (reordered / OLMo2 post-norm), :169-185 (Gemma pre+post)."""
    pre = f"layers.{l}."
    tape = {"x": x}
    an, mn = P[pre + "attention_norm.weight"], P[pre + "mlp_norm.weight"]
    if cfg.layer_type == "pre":
        a = _attn_fwd(cfg, P, pre, l, rms_norm_fwd(x, an, cfg.eps, rt), tape, rt)
        h = rt(x + a)
        m = _mlp_fwd(cfg, P, pre, rms_norm_fwd(h, mn, cfg.eps, rt), tape, rt)
        out = rt(h + m)
    elif cfg.layer_type == "reordered":
        a = _attn_fwd(cfg, P, pre, l, x, tape, rt)
        h = rt(x + rms_norm_fwd(a, an, cfg.eps, rt))
        m = _mlp_fwd(cfg, P, pre, h, tape, rt)
        out = rt(h + rms_norm_fwd(m, mn, cfg.eps, rt))
        tape.update(a_out=a, m_out=m)
    elif cfg.layer_type == "gemma":
        ain, minn = P[pre + "attention_input_norm.weight"], P[pre + "mlp_input_norm.weight"]
        a = _attn_fwd(cfg, P, pre, l, rms_norm_fwd(x, ain, cfg.eps, rt), tape, rt)
        h = rt(x + rms_norm_fwd(a, an, cfg.eps, rt))
        m = _mlp_fwd(cfg, P, pre, rms_norm_fwd(h, minn, cfg.eps, rt), tape, rt)
        out = rt(h + rms_norm_fwd(m, mn, cfg.eps, rt))
        tape.update(a_out=a, m_out=m)
    else:
        raise ValueError(cfg.layer_type)
    tape["h"] = h
    return out, tape


def block_bwd(cfg: ModelConfig, P: dict, l: int, dout: Tensor, tape: dict, G: dict, rt=_id):
    pre = f"layers.{l}."
    an, mn = P[pre + "attention_norm.weight"], P[pre + "mlp_norm.weight"]
    x, h = tape["x"], tape["h"]
    if cfg.layer_type == "pre":
        dmn = _mlp_bwd(cfg, P, pre, dout, tape, G, rt)
        dh_n, G[pre + "mlp_norm.weight"] = rms_norm_bwd(h, mn, dmn, cfg.eps, rt)
        dh = rt(dout + dh_n)
        dan = _attn_bwd(cfg, P, pre, l, dh, tape, G, rt)
        dx_n, G[pre + "attention_norm.weight"] = rms_norm_bwd(x, an, dan, cfg.eps, rt)
        return rt(dh + dx_n)
    if cfg.layer_type == "reordered":
        dm, G[pre + "mlp_norm.weight"] = rms_norm_bwd(tape["m_out"], mn, dout, cfg.eps, rt)
        dh = rt(dout + _mlp_bwd(cfg, P, pre, dm, tape, G, rt))
        da, G[pre + "attention_norm.weight"] = rms_norm_bwd(tape["a_out"], an, dh, cfg.eps, rt)
        return rt(dh + _attn_bwd(cfg, P, pre, l, da, tape, G, rt))
    # gemma
    ain, minn = P[pre + "attention_input_norm.weight"], P[pre + "mlp_input_norm.weight"]
    dm, G[pre + "mlp_norm.weight"] = rms_norm_bwd(tape["m_out"], mn, dout, cfg.eps, rt)
    dmi = _mlp_bwd(cfg, P, pre, dm, tape, G, rt)
    dh_n, G[pre + "mlp_input_norm.weight"] = rms_norm_bwd(h, minn, dmi, cfg.eps, rt)
    dh = rt(dout + dh_n)
    da, G[pre + "attention_norm.weight"] = rms_norm_bwd(tape["a_out"], an, dh, cfg.eps, rt)
    dai = _attn_bwd(cfg, P, pre, l, da, tape, G, rt)
    dx_n, G[pre + "attention_input_norm.weight"] = rms_norm_bwd(x, ain, dai, cfg.eps, rt)
    return rt(dh + dx_n)


def model_loss_and_grads(cfg: ModelConfig, P: dict, ids: Tensor, labels: Tensor, rt=_id):
    """Transformer.forward (src/olmax/nn/transformer/model.py:95-136) + cross_entropy_loss
    (src/integration_tests/train_transformer.py:190-206) and the full hand-derived backward.
    Returns (loss, grads dict keyed like P)."""
    G: dict = {}
    h = embed_fwd(ids, P["embedding.weight"])
    tapes = []
    for l in range(cfg.n_layers):
        h, tape = block_fwd(cfg, P, l, h, rt)
        tapes.append(tape)
    hn = rms_norm_fwd(h, P["norm.weight"], cfg.eps, rt)
    w_out = P["embedding.weight"] if cfg.tied else P["lm_head.proj.weight"]
    B, S, d = hn.shape
    loss, dhn, dw_out = lm_head_ce(hn.reshape(B * S, d), w_out, labels.reshape(-1),
                                   softcap=cfg.final_softcap, rt=rt)
    dh, G["norm.weight"] = rms_norm_bwd(h, P["norm.weight"], dhn.reshape(B, S, d), cfg.eps, rt)
    for l in reversed(range(cfg.n_layers)):
        dh = block_bwd(cfg, P, l, dh, tapes[l], G, rt)
    demb = embed_bwd(ids, dh, cfg.vocab)
    if cfg.tied:
        G["embedding.weight"] = rt(demb + dw_out)
    else:
        G["embedding.weight"] = rt(demb)
        G["lm_head.proj.weight"] = dw_out
    return loss, G


def decay_mask(names, no_decay) -> dict:
    """OptimConfig.build_weight_decay_mask (src/olmax/optim/config.py:94-122): a leaf decays
    unless its dotted path matches one of the fnmatch patterns."""
    return {n: not any(_fnmatch(n, pat) for pat in (no_decay or ())) for n in names}


def clip_by_global_norm(G: dict, max_norm: float):
    """clip_grads_by_global_norm (src/olmax/optim/utils.py:22-38; norm from get_global_norm,
    src/olmax/jax_utils.py:88-102): g <- (g / max(max_norm, ||g||)) * max_norm over ALL leaves
    together.  Returns (clipped, norm)."""
    norm = torch.sqrt(sum((g.double() ** 2).sum() for g in G.values()))
    clamped = max(float(max_norm), float(norm))
    return {n: (g / clamped) * max_norm for n, g in G.items()}, norm


def multisteps_mean(grads: list) -> dict:
    """optax.MultiSteps' accumulator (third party; built at src/olmax/optim/config.py:153-154):
    the k micro-batch gradients enter a running mean acc += (g - acc) / (j + 1)."""
    acc = None
    for j, G in enumerate(grads):
        acc = dict(G) if acc is None else {n: acc[n] + (G[n] - acc[n]) / (j + 1) for n in acc}
    return acc


def apply_adamw(master: dict, opt: dict, G: dict, *, step: int, lr: float, b1=0.9, b2=0.999, eps=1e-8,
                wd=1e-4, no_decay=("embedding.weight",)) -> None:
    """step_optimizer (src/olmax/train/trainer.py:742-757): optax.adamw with the weight-decay
    mask of AdamWConfig.build (src/olmax/optim/config.py:136-148) on every leaf, in place."""
    mask = decay_mask(master, no_decay)
    for name in master:
        master[name], opt["m"][name], opt["v"][name] = adamw_step(
            master[name], G[name].to(master[name].dtype), opt["m"][name], opt["v"][name],
            step=step, lr=lr, b1=b1, b2=b2, eps=eps, wd=wd if mask[name] else 0.0)


def _compute_params(master: dict, compute_bf16: bool):
    if compute_bf16:
        return {k: bf16_round(v) for k, v in master.items()}, bf16_round
    return master, _id


def train_step(cfg: ModelConfig, master: dict, opt: dict, ids, labels, *, step: int, lr: float,
               b1=0.9, b2=0.999, eps=1e-8, wd=1e-4, no_decay=("embedding.weight",),
               compute_bf16: bool = False):
    """process_microbatch (src/olmax/train/trainer.py:723-777): cast master → compute dtype,
    loss+grads, grads → fp32, AdamW on the fp32 master copy.  `opt` = {"m":…, "v":…}."""
    P, rt = _compute_params(master, compute_bf16)
    loss, G = model_loss_and_grads(cfg, P, ids, labels, rt)
    apply_adamw(master, opt, G, step=step, lr=lr, b1=b1, b2=b2, eps=eps, wd=wd, no_decay=no_decay)
    return loss, G


def train_batch(cfg: ModelConfig, master: dict, opt: dict, batch, *, step: int, lr: float,
                b1=0.9, b2=0.999, eps=1e-8, wd=1e-4, no_decay=("embedding.weight",),
                compute_bf16: bool = False, max_grad_norm=None):
    """train_batch (src/olmax/train/trainer.py:779-807) with the optimizer wrapped in
    optax.MultiSteps(k) (src/olmax/optim/config.py:153-154; third party, restated from its
    documentation): gradients are cast to fp32 (trainer.py:738), the k micro-batches enter the
    running mean, the clip (src/olmax/optim/utils.py:22-38) and AdamW act once, on the mean, and
    the reported loss is the mean of the micro-batch losses.  `batch` = [(ids, labels), ...]."""
    P, rt = _compute_params(master, compute_bf16)
    grads, losses = [], []
    for ids, labels in batch:
        loss, G = model_loss_and_grads(cfg, P, ids, labels, rt)
        losses.append(loss)
        grads.append({n: g.to(torch.float32).to(master[n].dtype) for n, g in G.items()})
    acc = multisteps_mean(grads)
    if max_grad_norm is not None:
        acc, _ = clip_by_global_norm(acc, max_grad_norm)
    apply_adamw(master, opt, acc, step=step, lr=lr, b1=b1, b2=b2, eps=eps, wd=wd, no_decay=no_decay)
    return sum(losses) / len(losses), acc


def _fnmatch(name: str, pat: str) -> bool:
    import fnmatch

    return fnmatch.fnmatch(name, pat)
