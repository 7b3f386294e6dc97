"""Pins the CPU oracle (oracle/ref.py) without the reference: closed forms, textbook
routines, invariants and autograd/finite differences, each chosen so that a dropped term,
wrong sign or transposed index fails.  The only reference-held known answers on this path
(the WSD schedule, src/test/optim/config_test.py:22-33, and the shapes of the sequential
token generator, src/test/data/utils_test.py) are reproduced literally."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import ref

torch.manual_seed(0)
D64 = torch.float64


def test_rms_norm_closed_form_and_invariants():
    x = torch.randn(5, 7, 16, dtype=D64)
    w = torch.randn(16, dtype=D64)
    y = ref.rms_norm_fwd(x, w, 1e-6)
    assert torch.allclose(y, F.rms_norm(x, (16,), w, 1e-6), atol=1e-12)
    y1 = ref.rms_norm_fwd(x, torch.ones(16, dtype=D64), 0.0)
    assert torch.allclose((y1 * y1).mean(-1), torch.ones(5, 7, dtype=D64), atol=1e-12)
    assert torch.allclose(ref.rms_norm_fwd(3.7 * x, w, 0.0), ref.rms_norm_fwd(x, w, 0.0), atol=1e-12)


def test_rms_norm_bwd_matches_autograd():
    x = torch.randn(4, 6, 32, dtype=D64, requires_grad=True)
    w = torch.randn(32, dtype=D64, requires_grad=True)
    dy = torch.randn(4, 6, 32, dtype=D64)
    y = F.rms_norm(x, (32,), w, 1e-5)
    gx, gw = torch.autograd.grad(y, (x, w), dy)
    dx, dw = ref.rms_norm_bwd(x.detach(), w.detach(), dy, 1e-5)
    assert torch.allclose(dx, gx, atol=1e-11) and torch.allclose(dw, gw, atol=1e-11)
    # eps = 0: dx is orthogonal to x
    dx0, _ = ref.rms_norm_bwd(x.detach(), w.detach(), dy, 0.0)
    assert (dx0 * x.detach()).sum(-1).abs().max() < 1e-10


def test_rope_properties():
    S, Dh = 24, 16
    cos, sin = ref.rope_tables(S, Dh, 10000.0, dtype=D64)
    assert cos.shape == (S, Dh // 2)
    # closed form of one entry
    assert abs(cos[5, 3].item() - math.cos(5 * 10000.0 ** (-6 / 16))) < 1e-12
    x = torch.randn(2, S, 3, Dh, dtype=D64)
    y = ref.rope_fwd(x, cos, sin)
    assert torch.allclose(y[:, 0], x[:, 0])  # position 0 is the identity
    # pairs (j, j + D/2) are rotated: their norm is preserved
    n_in = x[..., :8] ** 2 + x[..., 8:] ** 2
    n_out = y[..., :8] ** 2 + y[..., 8:] ** 2
    assert torch.allclose(n_in, n_out, atol=1e-12)
    # HF rotate_half convention, written out independently
    c2 = torch.cat([cos, cos], -1)[None, :, None, :]
    s2 = torch.cat([sin, sin], -1)[None, :, None, :]
    rot = torch.cat([-x[..., 8:], x[..., :8]], -1)
    assert torch.allclose(y, x * c2 + rot * s2, atol=1e-12)
    # relative-position property
    q = torch.randn(Dh, dtype=D64)
    k = torch.randn(Dh, dtype=D64)
    def at(vec, p):
        t = torch.zeros(1, S, 1, Dh, dtype=D64); t[0, p, 0] = vec
        return ref.rope_fwd(t, cos, sin)[0, p, 0]
    assert abs((at(q, 7) @ at(k, 3)) - (at(q, 14) @ at(k, 10))) < 1e-10
    # bwd == transpose
    xg = x.clone().requires_grad_(True)
    dy = torch.randn_like(x)
    (gx,) = torch.autograd.grad(ref.rope_fwd(xg, cos, sin), xg, dy)
    assert torch.allclose(ref.rope_bwd(dy, cos, sin), gx, atol=1e-12)


def test_linear_against_bruteforce():
    x = torch.randn(3, 5, dtype=D64); w = torch.randn(4, 5, dtype=D64); dy = torch.randn(3, 4, dtype=D64)
    y = ref.linear_fwd(x, w)
    for i in range(3):
        for o in range(4):
            assert abs(y[i, o] - sum(x[i, k] * w[o, k] for k in range(5))) < 1e-12
    dx, dw = ref.linear_bwd(x, w, dy)
    xg = x.clone().requires_grad_(True); wg = w.clone().requires_grad_(True)
    gx, gw = torch.autograd.grad(F.linear(xg, wg), (xg, wg), dy)
    assert torch.allclose(dx, gx) and torch.allclose(dw, gw)


@pytest.mark.parametrize("kind", ["silu", "gelu"])
def test_glu(kind):
    g = torch.randn(64, dtype=D64) * 3; u = torch.randn(64, dtype=D64); dh = torch.randn(64, dtype=D64)
    want = (F.silu(g) if kind == "silu" else F.gelu(g, approximate="tanh")) * u
    assert torch.allclose(ref.glu_fwd(g, u, kind), want, atol=1e-12)
    gg = g.clone().requires_grad_(True); ug = u.clone().requires_grad_(True)
    a = (F.silu(gg) if kind == "silu" else F.gelu(gg, approximate="tanh")) * ug
    eg, eu = torch.autograd.grad(a, (gg, ug), dh)
    dg, du = ref.glu_bwd(g, u, dh, kind)
    assert torch.allclose(dg, eg, atol=1e-11) and torch.allclose(du, eu, atol=1e-11)


def _attn_autograd(q, k, v, window, softcap):
    """Independent formulation (masked softmax via additive -inf bias, GQA by expand)."""
    B, S, H, Dh = q.shape
    K = k.shape[2]
    qh = q.permute(0, 2, 1, 3)
    kh = k.permute(0, 2, 1, 3)[:, :, None].expand(B, K, H // K, S, Dh).reshape(B, H, S, Dh)
    vh = v.permute(0, 2, 1, 3)[:, :, None].expand(B, K, H // K, S, Dh).reshape(B, H, S, Dh)
    s = qh @ kh.transpose(-1, -2) / math.sqrt(Dh)
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    bias = torch.zeros(S, S, dtype=q.dtype)
    for i in range(S):
        for j in range(S):
            if j > i or (window is not None and j < i - window):
                bias[i, j] = float("-inf")
    p = torch.softmax(s + bias, -1)
    return (p @ vh).permute(0, 2, 1, 3)


@pytest.mark.parametrize("H,K,window,softcap", [(4, 4, None, 0.0), (4, 2, None, 0.0), (4, 2, 5, 0.0), (4, 1, 3, 7.0), (2, 2, None, 2.5)])
def test_attention_fwd_bwd(H, K, window, softcap):
    B, S, Dh = 2, 17, 8
    q = torch.randn(B, S, H, Dh, dtype=D64, requires_grad=True)
    k = torch.randn(B, S, K, Dh, dtype=D64, requires_grad=True)
    v = torch.randn(B, S, K, Dh, dtype=D64, requires_grad=True)
    do = torch.randn(B, S, H, Dh, dtype=D64)
    want = _attn_autograd(q, k, v, window, softcap)
    gq, gk, gv = torch.autograd.grad(want, (q, k, v), do)
    o, lse = ref.attention_fwd(q.detach(), k.detach(), v.detach(), window=window, softcap=softcap)
    assert torch.allclose(o, want.detach(), atol=1e-11)
    assert torch.allclose(o[:, 0], v.detach().repeat_interleave(H // K, 2)[:, 0], atol=1e-12)  # first query sees key 0 only
    dq, dk, dv = ref.attention_bwd(q.detach(), k.detach(), v.detach(), o, lse, do, window=window, softcap=softcap)
    assert torch.allclose(dq, gq, atol=1e-10) and torch.allclose(dk, gk, atol=1e-10) and torch.allclose(dv, gv, atol=1e-10)


def test_attention_textbook_and_limits():
    B, S, H, K, Dh = 1, 12, 4, 2, 8
    q = torch.randn(B, S, H, Dh, dtype=D64); k = torch.randn(B, S, K, Dh, dtype=D64); v = torch.randn(B, S, K, Dh, dtype=D64)
    o, _ = ref.attention_fwd(q, k, v)
    want = F.scaled_dot_product_attention(q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3), v.permute(0, 2, 1, 3), is_causal=True, enable_gqa=True).permute(0, 2, 1, 3)
    assert torch.allclose(o, want, atol=1e-11)
    assert torch.allclose(ref.attention_fwd(q, k, v, window=S - 1)[0], o, atol=1e-12)  # window >= S-1 is full causal
    assert torch.allclose(ref.attention_fwd(q, k, v, softcap=1e9)[0], o, atol=1e-9)   # cap -> inf is no cap
    # window w keeps exactly w + 1 keys: with w = 0 every query sees only itself
    assert torch.allclose(ref.attention_fwd(q, k, v, window=0)[0], v.repeat_interleave(2, 2), atol=1e-12)
    assert ref.attention_mask(6, 2).sum(1).tolist() == [1, 2, 3, 3, 3, 3]


def test_cross_entropy():
    T, V = 9, 11
    logits = torch.randn(T, V, dtype=D64)
    labels = torch.randint(0, V, (T,))
    labels[2] = -100
    loss, lse, n = ref.cross_entropy_fwd(logits, labels)
    assert abs(loss - F.cross_entropy(logits, labels, ignore_index=-100)) < 1e-12
    from scipy.special import logsumexp
    assert abs(lse[3].item() - logsumexp(logits[3].numpy())) < 1e-12
    # reference invariant (src/test/nn/functional_test.py:10-18): an appended ignored row changes nothing
    l2, _, _ = ref.cross_entropy_fwd(torch.cat([logits, torch.randn(1, V, dtype=D64)]), torch.cat([labels, torch.tensor([-100])]))
    assert abs(l2 - loss) < 1e-12
    # uniform logits -> ln V
    assert abs(ref.cross_entropy_fwd(torch.zeros(4, V, dtype=D64), torch.tensor([0, 1, 2, 3]))[0] - math.log(V)) < 1e-12
    # bwd vs autograd, rows sum to zero
    lg = logits.clone().requires_grad_(True)
    (g,) = torch.autograd.grad(F.cross_entropy(lg, labels, ignore_index=-100), lg)
    d = ref.cross_entropy_bwd(logits, labels)
    assert torch.allclose(d, g, atol=1e-12)
    assert d.sum(-1).abs().max() < 1e-12 and d[2].abs().max() == 0


def test_cross_entropy_sum_and_none_reductions():
    """src/olmax/nn/functional.py:84-91 against torch's own reductions, forward and backward."""
    g = torch.Generator().manual_seed(4)
    T, V = 9, 23
    logits = torch.randn(T, V, generator=g, dtype=D64)
    labels = torch.randint(0, V, (T,), generator=g)
    labels[2] = -100
    for red in ("sum", "none"):
        got = ref.cross_entropy_fwd(logits, labels, reduction=red)[0]
        want = F.cross_entropy(logits, labels, ignore_index=-100, reduction=red)
        assert torch.allclose(got, want, atol=1e-12)
    lg = logits.clone().requires_grad_(True)
    (gs,) = torch.autograd.grad(F.cross_entropy(lg, labels, ignore_index=-100, reduction="sum") * 0.5, lg)
    assert torch.allclose(ref.cross_entropy_bwd(logits, labels, dloss=0.5, reduction="sum"), gs, atol=1e-12)
    w = torch.randn(T, generator=g, dtype=D64)
    (gn,) = torch.autograd.grad((F.cross_entropy(lg, labels, ignore_index=-100, reduction="none") * w).sum(), lg)
    assert torch.allclose(ref.cross_entropy_bwd(logits, labels, dloss=w, reduction="none"), gn, atol=1e-12)
    # out-of-range label (one_hot gives an all-zero row): zero loss and gradient in every reduction
    labels[4] = V
    per = ref.cross_entropy_fwd(logits, labels, reduction="none")[0]
    assert per[4] == 0 and per[2] == 0 and ref.cross_entropy_bwd(logits, labels, reduction="sum")[4].abs().max() == 0


def test_cross_entropy_out_of_range_label_quirk():
    """label == V (made by the synthetic loader when input == V-1): zero loss, zero grad, but
    the row still counts in the mean (one_hot gives zeros; `where` is labels != -100)."""
    V = 3
    logits = torch.tensor([[0.0, 0.0, 0.0], [1.0, 2.0, 3.0], [5.0, 5.0, 5.0]], dtype=D64)
    labels = torch.tensor([0, V, -100])
    loss, _, n = ref.cross_entropy_fwd(logits, labels)
    assert n == 2 and abs(loss - math.log(3) / 2) < 1e-12   # (ln3 + 0) / 2, hand computed
    d = ref.cross_entropy_bwd(logits, labels)
    assert torch.allclose(d[0], torch.tensor([1 / 3 - 1, 1 / 3, 1 / 3], dtype=D64) / 2)
    assert d[1].abs().max() == 0 and d[2].abs().max() == 0


def test_final_softcap_ce_matches_autograd():
    T, V, c = 6, 13, 3.0
    logits = torch.randn(T, V, dtype=D64) * 4
    labels = torch.randint(0, V, (T,))
    lg = logits.clone().requires_grad_(True)
    l = F.cross_entropy(c * torch.tanh(lg / c), labels)
    (g,) = torch.autograd.grad(l, lg)
    assert abs(ref.cross_entropy_fwd(logits, labels, softcap=c)[0] - l.detach()) < 1e-12
    assert torch.allclose(ref.cross_entropy_bwd(logits, labels, softcap=c), g, atol=1e-12)


def test_adamw_hand_example_and_torch():
    # 1 element, 2 steps, computed by hand: b1=.9 b2=.999 eps=1e-8 wd=.1 lr=.01, p0=1, g=(0.5, -0.25)
    p, m, v = torch.tensor([1.0], dtype=D64), torch.zeros(1, dtype=D64), torch.zeros(1, dtype=D64)
    p, m, v = ref.adamw_step(p, torch.tensor([0.5], dtype=D64), m, v, step=1, lr=0.01, wd=0.1)
    # step 1: mhat = g, vhat = g^2 -> update = sign(g) (+ wd p)
    assert abs(p.item() - (1 - 0.01 * (0.5 / (0.5 + 1e-8) + 0.1 * 1.0))) < 1e-15
    p1 = p.item()
    p, m, v = ref.adamw_step(p, torch.tensor([-0.25], dtype=D64), m, v, step=2, lr=0.01, wd=0.1)
    m2 = 0.9 * 0.05 + 0.1 * -0.25; v2 = 0.999 * 0.00025 + 0.001 * 0.0625
    want = p1 - 0.01 * ((m2 / (1 - 0.81)) / (math.sqrt(v2 / (1 - 0.999 ** 2)) + 1e-8) + 0.1 * p1)
    assert abs(p.item() - want) < 1e-15
    # g = 0 -> pure decay
    p0 = torch.tensor([2.0], dtype=D64)
    assert abs(ref.adamw_step(p0, torch.zeros(1, dtype=D64), torch.zeros(1, dtype=D64), torch.zeros(1, dtype=D64), step=1, lr=0.1, wd=0.5)[0].item() - 2.0 * (1 - 0.05)) < 1e-15
    # torch.optim.AdamW is algebraically the same update
    w = torch.randn(50, dtype=D64)
    tp = w.clone().requires_grad_(True)
    opt = torch.optim.AdamW([tp], lr=3e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    p, m, v = w.clone(), torch.zeros_like(w), torch.zeros_like(w)
    for t in range(1, 6):
        g = torch.randn(50, dtype=D64)
        tp.grad = g.clone(); opt.step()
        p, m, v = ref.adamw_step(p, g, m, v, step=t, lr=3e-3, b1=0.9, b2=0.95, wd=0.1)
    assert torch.allclose(p, tp.detach(), atol=1e-12)


def test_schedules_known_answers():
    # literal values of the reference's own test, src/test/optim/config_test.py:22-33
    r = [ref.wsd_lr(s, warmup_steps=10, stable_steps=10, decay_steps=10, peak=1.0) for s in range(31)]
    assert (r[0], r[5], r[10], r[20], r[25], r[30]) == (0.0, 0.5, 1.0, 1.0, 0.5, 0.0)
    kw = dict(warmup_steps=20, decay_steps=80, peak=1e-4, init=1e-6, end=1e-6)
    assert ref.warmup_cosine_lr(0, **kw) == 1e-6
    assert abs(ref.warmup_cosine_lr(20, **kw) - 1e-4) < 1e-18
    assert abs(ref.warmup_cosine_lr(60, **kw) - (1e-6 + (1e-4 - 1e-6) * 0.5)) < 1e-18
    assert abs(ref.warmup_cosine_lr(100, **kw) - 1e-6) < 1e-18


def test_sequential_tokens():
    ins, tg = ref.sequential_tokens(torch.tensor([0, 5, 9]), 8, 10)
    assert ins.shape == (3, 8) and ins.dtype == torch.int32
    assert ins[1].tolist() == [5, 6, 7, 8, 9, 0, 1, 2]
    assert tg[1].tolist() == [6, 7, 8, 9, 10, 1, 2, 3]  # target == V after input V-1


def test_embedding_scatter_add():
    ids = torch.tensor([[1, 3, 1]])
    dh = torch.arange(6, dtype=D64).reshape(1, 3, 2)
    dw = ref.embed_bwd(ids, dh, 5)
    assert dw[1].tolist() == [4.0, 6.0] and dw[3].tolist() == [2.0, 3.0] and dw[0].abs().sum() == 0


def _autograd_model_loss(cfg, P, ids, labels):
    """Forward only from the oracle's forward pieces; autograd supplies the gradients."""
    h = P["embedding.weight"][ids.long()]
    for l in range(cfg.n_layers):
        h, _ = ref.block_fwd(cfg, P, l, h)
    hn = ref.rms_norm_fwd(h, P["norm.weight"], cfg.eps)
    w = P["embedding.weight"] if cfg.tied else P["lm_head.proj.weight"]
    logits = hn @ w.t()
    return ref.cross_entropy_fwd(logits.reshape(-1, cfg.vocab), labels.reshape(-1), softcap=cfg.final_softcap)[0]


@pytest.mark.parametrize("kind", ["pre", "reordered", "gemma"])
def test_model_grads_match_autograd(kind):
    cfg = ref.ModelConfig(vocab=37, d_model=16, n_layers=2, n_heads=4, n_kv_heads=2 if kind == "gemma" else 4,
                          head_dim=4, hidden=24, layer_type=kind, act="gelu" if kind == "gemma" else "silu",
                          qk_norm=kind != "pre", qk_norm_headwise=kind != "reordered", windows=[3, None] if kind == "gemma" else None,
                          rope_theta_layers=[1e4, 1e6] if kind == "gemma" else None,
                          attn_softcap=5.0 if kind == "gemma" else 0.0, final_softcap=3.0 if kind == "gemma" else 0.0,
                          tied=kind == "gemma")
    P = {k: (v.double() * (10 if "norm" not in k else 1) + (0.1 * torch.randn_like(v.double()) if "norm" in k else 0)).requires_grad_(True)
         for k, v in ref.init_params(cfg, seed=1).items()}
    ids = torch.randint(0, cfg.vocab, (2, 9)); labels = torch.randint(0, cfg.vocab, (2, 9)); labels[0, 2] = -100; labels[1, 1] = cfg.vocab
    loss = _autograd_model_loss(cfg, P, ids, labels)
    names = list(P)
    grads = torch.autograd.grad(loss, [P[n] for n in names])
    Pd = {k: v.detach() for k, v in P.items()}
    loss2, G = ref.model_loss_and_grads(cfg, Pd, ids, labels)
    assert abs(loss2 - loss.detach()) < 1e-12
    for n, g in zip(names, grads):
        assert torch.allclose(G[n], g, atol=1e-10, rtol=1e-8), n


def test_train_step_decreases_loss():
    cfg = ref.ModelConfig(vocab=50, d_model=16, n_layers=1, n_heads=2, n_kv_heads=2, head_dim=8, hidden=32)
    master = ref.init_params(cfg, seed=0)
    opt = {"m": {k: torch.zeros_like(v) for k, v in master.items()}, "v": {k: torch.zeros_like(v) for k, v in master.items()}}
    ids = torch.randint(0, 50, (2, 8)); labels = torch.randint(0, 50, (2, 8))
    losses = [ref.train_step(cfg, master, opt, ids, labels, step=s, lr=1e-2, wd=0.1)[0].item() for s in range(1, 6)]
    assert losses[-1] < losses[0]


# ------------------------------------------------------------------------------------------
# Pins for the pieces that used to be checked only against themselves: fp32 RoPE tables, the
# three residual orderings, the weight-decay mask, global-norm clipping, the micro-batch
# running mean and train_batch as a whole.  Each expected value below is built WITHOUT the
# oracle function under test: closed forms, hand arithmetic, or torch's own textbook routines
# (F.rms_norm, F.linear, F.scaled_dot_product_attention, torch.optim.AdamW, autograd).
# ------------------------------------------------------------------------------------------
def test_rope_tables_fp32_follow_reference_arithmetic():
    """src/olmax/nn/rope.py:127-133 forms freqs, t and the outer product in fp32.  Against the
    exact closed form cos(p * theta^(-2i/D)) the fp32 table may be off by the rounding of the
    angle: |d angle| <= 4 ulp(fp32) of the angle (pow, reciprocal, product), i.e.
    4 * 2^-23 * angle, plus the fp32 rounding of cos/sin itself."""
    S, Dh, theta = 4096, 128, 500000.0
    cos, sin = ref.rope_tables(S, Dh, theta)
    assert cos.dtype == torch.float32 and cos.shape == (S, Dh // 2)
    p = torch.arange(S, dtype=D64)[:, None]
    i = torch.arange(Dh // 2, dtype=D64)[None, :]
    ang = p * theta ** (-2.0 * i / Dh)
    tol = 4 * 2.0 ** -23 * ang + 2.0 ** -23
    assert ((cos.double() - torch.cos(ang)).abs() <= tol).all()
    assert ((sin.double() - torch.sin(ang)).abs() <= tol).all()
    # the tolerance is tight enough to tell fp32 angles from a dropped or doubled exponent:
    wrong = p * theta ** (-1.0 * i / Dh)
    assert ((cos.double() - torch.cos(wrong)).abs() > tol).any()
    # frequency 0 has inv_freq == 1 exactly, so its angle is the integer position itself
    assert torch.equal(cos[:, 0], torch.cos(torch.arange(S, dtype=torch.float32)))
    assert torch.equal(cos[0], torch.ones(Dh // 2)) and torch.equal(sin[0], torch.zeros(Dh // 2))
    # and the fp32 table is NOT the fp64 table rounded (the reference's angles carry fp32 error)
    c64, _ = ref.rope_tables(S, Dh, theta, dtype=D64)
    assert (cos.double() - c64).abs().max() > 1e-5


def _torch_block(kind, P, pre, x, *, H, K, Dh, eps, theta, act, qk, window=None):
    """One transformer block written from the reference's three forward() bodies
    (src/olmax/nn/transformer/layer.py:86,90 / 108,112 / 175-177,181) and
    MultiheadSelfAttention.forward (src/olmax/nn/attention.py:270-317) with torch's own
    routines only; RoPE as a complex rotation of the (j, j + D/2) pairs."""
    B, S, _ = x.shape

    def norm(t, name):
        return F.rms_norm(t, (t.shape[-1],), P[pre + name], eps)

    def rope(t):
        pos = torch.arange(S, dtype=D64)[:, None]
        inv = theta ** (-torch.arange(0, Dh, 2, dtype=D64) / Dh)[None, :]
        z = torch.polar(torch.ones(S, Dh // 2, dtype=D64), pos * inv)
        tc = torch.complex(t[..., : Dh // 2], t[..., Dh // 2:]) * z[None, :, None, :]
        return torch.cat([tc.real, tc.imag], -1)

    def attn(t):
        q = F.linear(t, P[pre + "attention.q_proj.weight"])
        k = F.linear(t, P[pre + "attention.k_proj.weight"])
        v = F.linear(t, P[pre + "attention.v_proj.weight"]).reshape(B, S, K, Dh)
        if qk == "full":
            q, k = norm(q, "attention.q_norm.weight"), norm(k, "attention.k_norm.weight")
        q, k = q.reshape(B, S, H, Dh), k.reshape(B, S, K, Dh)
        if qk == "head":
            q, k = norm(q, "attention.q_norm.weight"), norm(k, "attention.k_norm.weight")
        q, k = rope(q), rope(k)
        if window is None:
            kw = dict(is_causal=True)
        else:  # keys i - window .. i (jax.nn.dot_product_attention's local_window_size=(window, 0) under is_causal)
            i, j = torch.arange(S)[:, None], torch.arange(S)[None, :]
            kw = dict(attn_mask=(j <= i) & (j >= i - window))
        o = F.scaled_dot_product_attention(q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3), v.permute(0, 2, 1, 3),
                                           enable_gqa=True, **kw).permute(0, 2, 1, 3)
        return F.linear(o.reshape(B, S, H * Dh), P[pre + "attention.o_proj.weight"])

    def mlp(t):
        g = F.linear(t, P[pre + "mlp.gate_proj.weight"])
        a = F.silu(g) if act == "silu" else F.gelu(g, approximate="tanh")
        return F.linear(a * F.linear(t, P[pre + "mlp.up_proj.weight"]), P[pre + "mlp.down_proj.weight"])

    if kind == "pre":
        h = x + attn(norm(x, "attention_norm.weight"))
        return h + mlp(norm(h, "mlp_norm.weight"))
    if kind == "reordered":
        h = x + norm(attn(x), "attention_norm.weight")
        return h + norm(mlp(h), "mlp_norm.weight")
    h = x + norm(attn(norm(x, "attention_input_norm.weight")), "attention_norm.weight")
    return h + norm(mlp(norm(h, "mlp_input_norm.weight")), "mlp_norm.weight")


def _random_block_params(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    P = {}
    for k, v in ref.init_params(cfg, seed=seed).items():
        v = v.double()
        P[k] = (1.0 + 0.3 * torch.randn(v.shape, generator=g, dtype=D64)) if "norm" in k else v * 10
    return P


@pytest.mark.parametrize("kind,qk", [("pre", "none"), ("pre", "full"), ("reordered", "head"), ("reordered", "none"),
                                     ("gemma", "head"), ("gemma", "full")])
def test_block_orderings_against_independent_torch_block(kind, qk):
    H, K = (4, 4) if qk == "full" or kind == "pre" else (4, 2)
    cfg = ref.ModelConfig(vocab=11, d_model=24, n_layers=2, n_heads=H, n_kv_heads=K, head_dim=6, hidden=40,
                          layer_type=kind, act="gelu" if kind == "gemma" else "silu", qk_norm=qk != "none",
                          qk_norm_headwise=qk != "full", eps=1e-5, rope_theta=777.0)
    P = _random_block_params(cfg, seed=3)
    x = torch.randn(2, 13, 24, dtype=D64)
    for l in range(2):
        want = _torch_block(kind, P, f"layers.{l}.", x, H=H, K=K, Dh=6, eps=1e-5, theta=777.0, act=cfg.act, qk=qk)
        got, _ = ref.block_fwd(cfg, P, l, x)
        # the oracle's block takes its cos/sin from the fp32 tables (as the reference does): 6e-8 relative
        assert torch.allclose(got, want, atol=2e-6), (kind, qk, (got - want).abs().max())
    # the three orderings are genuinely different functions of the same weights
    if qk == "none" and kind != "gemma":
        other = _torch_block("reordered" if kind == "pre" else "pre", P, "layers.0.", x, H=H, K=K, Dh=6, eps=1e-5,
                             theta=777.0, act=cfg.act, qk=qk)
        assert (ref.block_fwd(cfg, P, 0, x)[0] - other).abs().max() > 1e-3


def test_per_layer_theta_and_window_reach_the_right_layer():
    """cfg.theta(l) / cfg.window(l) inside ref.block_fwd: two Gemma layers with different RoPE
    bases, the first with a 5-key window, the second global (GemmaTransformerLayer,
    src/olmax/nn/transformer/layer.py:169-185; per-layer tables as RotaryEmbedding builds them,
    src/olmax/nn/rope.py:118-145), each against the independent torch block given that layer's own
    theta and window - and NOT equal to the block built with the other layer's settings."""
    cfg = ref.ModelConfig(vocab=11, d_model=24, n_layers=2, n_heads=4, n_kv_heads=2, head_dim=6, hidden=40,
                          layer_type="gemma", act="gelu", qk_norm=True, qk_norm_headwise=True, eps=1e-5, rope_theta=123.0,
                          rope_theta_layers=[50.0, 9000.0], windows=[4, None])
    P = _random_block_params(cfg, seed=8)
    x = torch.randn(2, 13, 24, dtype=D64)
    settings = [(50.0, 4), (9000.0, None)]
    for l, (theta, window) in enumerate(settings):
        kw = dict(H=4, K=2, Dh=6, eps=1e-5, act="gelu", qk="head")
        want = _torch_block("gemma", P, f"layers.{l}.", x, theta=theta, window=window, **kw)
        got, _ = ref.block_fwd(cfg, P, l, x)
        assert torch.allclose(got, want, atol=2e-6), (l, (got - want).abs().max())
        o_theta, o_window = settings[1 - l]
        assert (got - _torch_block("gemma", P, f"layers.{l}.", x, theta=o_theta, window=window, **kw)).abs().max() > 1e-3
        assert (got - _torch_block("gemma", P, f"layers.{l}.", x, theta=theta, window=o_window, **kw)).abs().max() > 1e-3
    # a window of w shows w + 1 keys: w = 3 differs from w = 4 at 13 tokens
    assert (_torch_block("gemma", P, "layers.0.", x, theta=50.0, window=3, H=4, K=2, Dh=6, eps=1e-5, act="gelu", qk="head")
            - ref.block_fwd(cfg, P, 0, x)[0]).abs().max() > 1e-4


def test_block_ordering_scale_invariants():
    """With eps = 0 a post-norm makes the block blind to the scale of o_proj / down_proj
    (layer.py:108,112,175,181: the norm sits AFTER the sub-layer); in the pre-norm block
    (layer.py:86,90) the sub-layer output is added as is, so its contribution scales."""
    x = torch.randn(1, 9, 16, dtype=D64)
    outs = {}
    for kind in ("pre", "reordered", "gemma"):
        cfg = ref.ModelConfig(vocab=5, d_model=16, n_layers=1, n_heads=2, n_kv_heads=2, head_dim=8, hidden=24,
                              layer_type=kind, eps=0.0)
        P = _random_block_params(cfg, seed=5)
        y1, t1 = ref.block_fwd(cfg, P, 0, x)
        P2 = dict(P)
        P2["layers.0.attention.o_proj.weight"] = 3.0 * P["layers.0.attention.o_proj.weight"]
        y2, t2 = ref.block_fwd(cfg, P2, 0, x)
        outs[kind] = (y1, y2, t1["h"], t2["h"])
    for kind in ("reordered", "gemma"):
        y1, y2, _, _ = outs[kind]
        assert torch.allclose(y1, y2, atol=1e-10), kind
    _, _, h1, h2 = outs["pre"]
    assert torch.allclose(h2 - x, 3.0 * (h1 - x), atol=1e-10)  # h = x + attn(...): linear in o_proj


def test_decay_mask_patterns_and_pure_decay():
    # the reference's own mask test (src/test/optim/config_test.py:36-47), names written out
    names = [f"{m}.{p}" for m in ("gate_proj", "up_proj", "down_proj") for p in ("weight", "bias")]
    mask = ref.decay_mask(names, ["gate_proj.bias", "down_proj.bias", "up_proj.bias"])
    assert all(mask[f"{m}.weight"] is True and mask[f"{m}.bias"] is False for m in ("gate_proj", "up_proj", "down_proj"))
    cfg = ref.ModelConfig(vocab=7, d_model=8, n_layers=2, n_heads=2, n_kv_heads=1, head_dim=4, hidden=12,
                          layer_type="gemma", qk_norm=True)
    master = {k: torch.full_like(v, 2.0).double() for k, v in ref.init_params(cfg).items()}
    mask = ref.decay_mask(master, ["embedding.weight", "*norm.weight"])
    assert mask["embedding.weight"] is False and mask["norm.weight"] is False
    assert mask["layers.1.attention.q_norm.weight"] is False and mask["layers.0.mlp_input_norm.weight"] is False
    assert mask["layers.0.mlp.up_proj.weight"] is True and mask["lm_head.proj.weight"] is True
    assert sum(not v for v in mask.values()) == 2 + 2 * 6
    # zero gradient: a masked leaf does not move, an unmasked one is p (1 - lr wd) exactly
    opt = {"m": {k: torch.zeros_like(v) for k, v in master.items()}, "v": {k: torch.zeros_like(v) for k, v in master.items()}}
    G = {k: torch.zeros_like(v) for k, v in master.items()}
    ref.apply_adamw(master, opt, G, step=1, lr=0.1, wd=0.25, no_decay=["embedding.weight", "*norm.weight"])
    for n, p in master.items():
        want = 2.0 if not mask[n] else 2.0 * (1 - 0.1 * 0.25)
        assert torch.equal(p, torch.full_like(p, want)), n


def test_clip_by_global_norm_hand_examples():
    """src/olmax/optim/utils.py:22-38: g * max_norm / max(max_norm, ||g||), one norm over all leaves."""
    G = {"a": torch.tensor([3.0, 0.0], dtype=D64), "b": torch.tensor([[4.0]], dtype=D64)}  # ||g|| = 5
    out, norm = ref.clip_by_global_norm(G, 1.0)
    assert abs(float(norm) - 5.0) < 1e-15
    assert torch.allclose(out["a"], torch.tensor([0.6, 0.0], dtype=D64), atol=1e-15) and abs(out["b"].item() - 0.8) < 1e-15
    out, norm = ref.clip_by_global_norm(G, 10.0)  # below the threshold: factor 10 / max(10, 5) = 1
    assert torch.allclose(out["a"], G["a"], atol=1e-15) and torch.allclose(out["b"], G["b"], atol=1e-15) and abs(float(norm) - 5.0) < 1e-15
    out, _ = ref.clip_by_global_norm(G, 5.0)      # exactly at the threshold
    assert torch.allclose(out["a"], G["a"], atol=1e-15)


def test_multisteps_running_mean_is_the_plain_mean():
    gs = [{"w": torch.tensor([1.0, -2.0], dtype=D64)}, {"w": torch.tensor([4.0, 0.0], dtype=D64)},
          {"w": torch.tensor([-2.0, 8.0], dtype=D64)}, {"w": torch.tensor([5.0, 2.0], dtype=D64)}]
    acc = ref.multisteps_mean(gs)
    assert torch.allclose(acc["w"], torch.tensor([2.0, 2.0], dtype=D64), atol=1e-15)  # (1+4-2+5)/4, (-2+0+8+2)/4
    assert torch.equal(ref.multisteps_mean(gs[:1])["w"], gs[0]["w"])


def _tiny_train_setup(dtype):
    cfg = ref.ModelConfig(vocab=23, d_model=16, n_layers=2, n_heads=2, n_kv_heads=1, head_dim=8, hidden=24,
                          layer_type="gemma", act="gelu", qk_norm=True, tied=False)
    g = torch.Generator().manual_seed(11)
    master = {}
    for k, v in ref.init_params(cfg, seed=2).items():
        master[k] = ((1.0 + 0.2 * torch.randn(v.shape, generator=g)) if "norm" in k else v * 8).to(dtype)
    batch = []
    for j in range(3):
        ids = torch.randint(0, 23, (2, 7), generator=g)
        labels = torch.randint(0, 23, (2, 7), generator=g)
        labels[0, : 2 * j] = -100  # different numbers of counted tokens per micro-batch
        batch.append((ids, labels))
    return cfg, master, batch


def _zeros_like_opt(master):
    return {"m": {k: torch.zeros_like(v) for k, v in master.items()}, "v": {k: torch.zeros_like(v) for k, v in master.items()}}


def test_train_batch_of_identical_microbatches_equals_train_step():
    cfg, master, batch = _tiny_train_setup(torch.float32)
    m1 = {k: v.clone() for k, v in master.items()}
    m2 = {k: v.clone() for k, v in master.items()}
    o1, o2 = _zeros_like_opt(m1), _zeros_like_opt(m2)
    ids, labels = batch[1]
    l1, _ = ref.train_step(cfg, m1, o1, ids, labels, step=1, lr=1e-2, wd=0.1)
    l2, _ = ref.train_batch(cfg, m2, o2, [(ids, labels)] * 3, step=1, lr=1e-2, wd=0.1)
    assert torch.equal(l1, l2)
    for n in m1:
        assert torch.equal(m1[n], m2[n]) and torch.equal(o1["v"][n], o2["v"][n]), n


@pytest.mark.parametrize("max_norm", [None, 0.05, 1e6])
def test_train_batch_against_autograd_and_torch_adamw(max_norm):
    """trainer.py:779-807 + optax.MultiSteps + the clip + masked AdamW, against a composition
    that shares nothing with it: by linearity the mean of the micro-batch gradients is the
    gradient of the mean of the micro-batch losses (autograd), the clip factor is computed by
    hand, and torch.optim.AdamW (two param groups: decayed / not decayed) takes the step."""
    cfg, master, batch = _tiny_train_setup(D64)
    no_decay = ["embedding.weight", "*norm.weight"]
    # --- independent composition
    P = {k: v.clone().requires_grad_(True) for k, v in master.items()}
    losses = [_autograd_model_loss(cfg, P, ids, labels) for ids, labels in batch]
    mean_loss = sum(losses) / 3
    names = list(P)
    grads = dict(zip(names, torch.autograd.grad(mean_loss, [P[n] for n in names])))
    norm = math.sqrt(sum(float((g ** 2).sum()) for g in grads.values()))
    factor = 1.0 if max_norm is None else max_norm / max(max_norm, norm)
    if max_norm == 0.05:
        assert norm > 0.05  # the clip really binds in this case
    import fnmatch
    nd = [n for n in names if any(fnmatch.fnmatch(n, p) for p in no_decay)]
    opt = torch.optim.AdamW([{"params": [P[n] for n in names if n not in nd], "weight_decay": 0.1},
                             {"params": [P[n] for n in nd], "weight_decay": 0.0}], lr=1e-2, betas=(0.9, 0.95), eps=1e-3)
    for n in names:
        P[n].grad = grads[n] * factor
    opt.step()
    # --- the oracle
    m2 = {k: v.clone() for k, v in master.items()}
    o2 = _zeros_like_opt(m2)
    loss, acc = ref.train_batch(cfg, m2, o2, batch, step=1, lr=1e-2, b1=0.9, b2=0.95, eps=1e-3, wd=0.1, no_decay=no_decay,
                                max_grad_norm=max_norm)
    assert abs(float(loss) - float(mean_loss.detach())) < 1e-7
    for n in names:
        # the oracle rounds gradients to fp32 (trainer.py:738) and rotates with fp32 cos/sin tables:
        # ~1e-7 of the largest gradient; eps = 1e-3 keeps the Adam step Lipschitz (lr / eps = 10) in g
        assert torch.allclose(acc[n], grads[n] * factor, rtol=1e-6, atol=1e-7), n
        assert torch.allclose(m2[n], P[n].detach(), atol=2e-6), (n, (m2[n] - P[n].detach()).abs().max())
    # and a second step, so that the moments carried in `opt` are exercised too
    losses = [_autograd_model_loss(cfg, P, ids, labels) for ids, labels in batch]
    grads = dict(zip(names, torch.autograd.grad(sum(losses) / 3, [P[n] for n in names])))
    norm = math.sqrt(sum(float((g ** 2).sum()) for g in grads.values()))
    factor = 1.0 if max_norm is None else max_norm / max(max_norm, norm)
    for n in names:
        P[n].grad = grads[n] * factor
    opt.step()
    ref.train_batch(cfg, m2, o2, batch, step=2, lr=1e-2, b1=0.9, b2=0.95, eps=1e-3, wd=0.1, no_decay=no_decay, max_grad_norm=max_norm)
    for n in names:
        assert torch.allclose(m2[n], P[n].detach(), atol=4e-6), (n, (m2[n] - P[n].detach()).abs().max())


def test_train_step_against_autograd_and_torch_adamw():
    """process_microbatch (trainer.py:723-777) in fp32 master / fp32 compute: same independent
    composition with one micro-batch and the benchmark's mask (embedding.weight only)."""
    cfg, master, batch = _tiny_train_setup(D64)
    ids, labels = batch[2]
    P = {k: v.clone().requires_grad_(True) for k, v in master.items()}
    names = list(P)
    opt = torch.optim.AdamW([{"params": [P[n] for n in names if n != "embedding.weight"], "weight_decay": 0.1},
                             {"params": [P["embedding.weight"]], "weight_decay": 0.0}], lr=3e-3, betas=(0.9, 0.999), eps=1e-8)
    m2 = {k: v.clone() for k, v in master.items()}
    o2 = _zeros_like_opt(m2)
    for step in (1, 2, 3):
        loss = _autograd_model_loss(cfg, P, ids, labels)
        for n, g in zip(names, torch.autograd.grad(loss, [P[n] for n in names])):
            P[n].grad = g
        opt.step()
        l2, _ = ref.train_step(cfg, m2, o2, ids, labels, step=step, lr=3e-3, wd=0.1)
        assert abs(float(l2) - float(loss.detach())) < 1e-7
    for n in names:
        assert torch.allclose(m2[n], P[n].detach(), atol=1e-5), n  # sign-like steps of 3e-3: any wrong term is >= 1e-3
