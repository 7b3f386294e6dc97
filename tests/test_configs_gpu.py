"""BASELINE configurations at their REAL widths on the GPU.

The CPU oracle cannot run 8192 tokens at these widths, so parity uses causality: with the
upstream gradient (or the labels) non-zero only on the first P tokens of sequence 0, the loss,
every weight gradient and dx[:P] depend on those P tokens alone, and the oracle is run on
exactly that prefix with the same weights.  Everything else is checked through
size-independent properties (zero rows stay zero, recompute == no recompute, loss at init)."""
import math

import pytest
import torch

from oracle import ref

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
rt = ref.bf16_round
P = 192  # prefix length checked against the oracle


def say(msg):
    print(f"[case] {msg}", flush=True)


def cosine(a, b):
    a, b = a.double().cpu().flatten(), b.double().cpu().flatten()
    return (a @ b / (a.norm() * b.norm() + 1e-30)).item()


def relerr(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).norm() / (b.norm() + 1e-30)).item()


def test_config2_olmo2_block_full_size():
    """One OLMo2-7B block (d 4096, 32x128 heads, SwiGLU 11008, post-norm + head-wise QK-norm,
    theta 5e5), activations [2, 4096, 4096], forward + backward."""
    say("config 2: OLMo2 block at full size")
    from olmax_amd import TransformerConfig
    from olmax_amd.layer import TransformerBlock
    B, S, d = 2, 4096, 4096
    hcfg = TransformerConfig(vocab_size=8, d_model=d, hidden_size=11008, num_layers=1, n_heads=32,
                             layer_type="reordered_norm", qk_norm_headwise=True, norm_eps=1e-6, rope_theta=5e5)
    ocfg = ref.ModelConfig(vocab=8, d_model=d, n_layers=1, n_heads=32, n_kv_heads=32, head_dim=128, hidden=11008,
                           layer_type="reordered", qk_norm=True, eps=1e-6, rope_theta=5e5)
    Pm = {k.replace("layers.0.", ""): rt(v) for k, v in ref.init_params(ocfg, seed=3).items() if k.startswith("layers.0.")}
    g = torch.Generator().manual_seed(4)
    for k in Pm:
        if "norm" in k:
            Pm[k] = rt(Pm[k] + 0.05 * torch.randn(Pm[k].shape, generator=g))
    blk = TransformerBlock(hcfg, batch_size=B, sequence_length=S)
    blk.load_state_dict(Pm)
    x = torch.randn(B, S, d, generator=g).to(BF)
    dy = torch.zeros(B, S, d, dtype=BF)
    dy[0, :P] = torch.randn(P, d, generator=g).to(BF)
    y = blk.forward(x.cuda().reshape(B * S, d))
    dx = blk.backward(dy.cuda().reshape(B * S, d)).reshape(B, S, d)
    # oracle on the prefix of sequence 0 (fp32 container, bf16 rounding points)
    Pd = {"layers.0." + k: v.float() for k, v in Pm.items()}
    wy, tape = ref.block_fwd(ocfg, Pd, 0, x[:1, :P].float(), rt)
    G = {}
    wdx = ref.block_bwd(ocfg, Pd, 0, dy[:1, :P].float(), tape, G, rt)
    assert relerr(y.reshape(B, S, d)[0, :P], wy[0]) < 1e-2
    assert cosine(dx[0, :P], wdx[0]) >= 0.999
    for n, gg in blk.grads.items():
        assert cosine(gg, G["layers.0." + n]) >= 0.999, n
    # rows whose upstream gradient is zero and that no later token attends to... sequence 1 gets nothing
    assert dx[1].abs().max().item() == 0.0
    assert dx[0, P:].abs().max().item() == 0.0
    # second forward of sequence 1 prefix agrees with the oracle too (both batch rows computed)
    wy1, _ = ref.block_fwd(ocfg, Pd, 0, x[1:, :64].float(), rt)
    assert relerr(y.reshape(B, S, d)[1, :64], wy1[0]) < 1e-2


def _model_prefix_check(hcfg, ocfg, B, S, seed, steps_adamw=False):
    from olmax_amd import AdamWConfig, ConstantSchedule, Trainer
    g = torch.Generator().manual_seed(seed)
    model = hcfg.build(batch_size=B, sequence_length=S, seed=seed)
    named = model.named_parameters()
    # perturb the norm weights so that their gradients matter, then read the weights back for the oracle
    for n, p in named.items():
        if "norm" in n:
            p.add_(0.05 * torch.randn(p.shape, generator=g).to(p.device))
    model.sync_working_copy()
    Pd = {n: p.detach().to(BF).float().cpu() for n, p in model.named_parameters().items()}
    ids = torch.randint(0, hcfg.vocab_size, (B, S), generator=g, dtype=torch.int32)
    labels = torch.full((B, S), -100, dtype=torch.int32)
    labels[0, :P] = torch.randint(0, hcfg.vocab_size, (P,), generator=g, dtype=torch.int32)
    labels[0, 5] = hcfg.vocab_size  # out-of-range label: zero loss and gradient, still counted
    loss = model.loss_and_grads(ids.cuda().reshape(-1), labels.cuda().reshape(-1)).item()
    G = model.named_gradients()
    wloss, WG = ref.model_loss_and_grads(ocfg, Pd, ids[:1, :P], labels[:1, :P].long(), rt)
    assert abs(loss - wloss.item()) < 1e-2 * abs(wloss.item()), (loss, wloss.item())
    worst = min((cosine(G[n], WG[n]), n) for n in G)
    assert worst[0] >= 0.999, worst
    return model, loss


def test_config4_gemma2_slice_full_width():
    """Gemma2-27B-like 4-layer slice: d 4608, 32/16 heads x 128, GeGLU 36864, pre+post norm,
    alternating 4096-window / global layers, attention soft-cap 50, final soft-cap 30, vocab
    256000 tied; seq 4096, micro-batch 2."""
    say("config 4: Gemma2 slice at full width")
    from olmax_amd import TransformerConfig
    L = 4
    hcfg = TransformerConfig(vocab_size=256000, d_model=4608, hidden_size=36864, num_layers=L, n_heads=32, n_kv_heads=16,
                             head_dim=128, layer_type="gemma", activation="gelu", norm_eps=1e-6, rope_theta=1e4,
                             window_size_per_layer=[4096, None, 4096, None], attn_logit_softcap=50.0,
                             final_logit_softcap=30.0, tie_embeddings=True, layer_ac_policy="nothing_saveable")
    ocfg = ref.ModelConfig(vocab=256000, d_model=4608, n_layers=L, n_heads=32, n_kv_heads=16, head_dim=128, hidden=36864,
                           layer_type="gemma", act="gelu", eps=1e-6, rope_theta=1e4, windows=[4096, None, 4096, None],
                           attn_softcap=50.0, final_softcap=30.0, tied=True)
    model, loss = _model_prefix_check(hcfg, ocfg, 2, 4096, seed=11)
    assert abs(loss - math.log(256000)) < 1.0  # near-uniform prediction at init


def test_config5_gemma3_slice_full_width_with_adamw():
    """Gemma3-27B-like 6-layer slice (5 local : 1 global): d 5376, 32/16 heads x 128, QK-norm,
    1024-token windows, theta 1e4 local / 1e6 global, GeGLU 21504, vocab 262144 tied; fwd+bwd
    and a fused AdamW step."""
    say("config 5: Gemma3 slice at full width")
    from olmax_amd import TransformerConfig
    L = 6
    win = [1024] * 5 + [None]
    th = [1e4] * 5 + [1e6]
    hcfg = TransformerConfig(vocab_size=262144, d_model=5376, hidden_size=21504, num_layers=L, n_heads=32, n_kv_heads=16,
                             head_dim=128, layer_type="gemma", activation="gelu", qk_norm_headwise=True, norm_eps=1e-6,
                             rope_theta_per_layer=th, window_size_per_layer=win, tie_embeddings=True,
                             layer_ac_policy="nothing_saveable")
    ocfg = ref.ModelConfig(vocab=262144, d_model=5376, n_layers=L, n_heads=32, n_kv_heads=16, head_dim=128, hidden=21504,
                           layer_type="gemma", act="gelu", qk_norm=True, eps=1e-6, rope_theta_layers=th, windows=win, tied=True)
    model, loss = _model_prefix_check(hcfg, ocfg, 2, 4096, seed=12)
    # The fused AdamW step of this configuration against the oracle (optax.adamw as built at
    # src/olmax/optim/config.py:136-148): two steps on the gradients just computed, weight decay
    # on, the embedding and every norm weight masked; master, m, v compared on sampled slices of
    # three leaves (a matrix with bf16 gradients, a masked norm weight and the masked, tied
    # embedding, both with fp32 gradients) after the SECOND step (non-zero moments, both bias
    # corrections != 1).
    pats = ["embedding.weight", "*norm.weight"]
    picks = {"layers.3.mlp.down_proj.weight": 0.05, "layers.0.attention.k_proj.weight": 0.05,
             "layers.4.attention.q_norm.weight": 0.0, "embedding.weight": 0.0}  # leaf -> the decay it must see
    leaves = {model.leaf_name(l): l for l in model.leaves}
    G = model.named_gradients()
    want, before = {}, {}
    gidx = torch.Generator().manual_seed(5)
    for n, wd in picks.items():
        l = leaves[n]
        idx = torch.randint(0, l.numel, (min(l.numel, 50_000),), generator=gidx).cuda()
        p = model.master[l.offset: l.offset + l.numel][idx].double().cpu()
        before[n] = p.clone()
        g = G[n].reshape(-1)[idx].double().cpu()
        assert g.abs().max().item() > 0, n
        m, v = torch.zeros_like(p), torch.zeros_like(p)
        for step in (1, 2):
            p, m, v = ref.adamw_step(p, g, m, v, step=step, lr=1e-3, b1=0.9, b2=0.95, eps=1e-8, wd=wd)
        want[n] = (idx, p, m, v)
    model.init_optimizer_state()
    for step in (1, 2):
        model.adamw_step(step=step, lr=1e-3, b1=0.9, b2=0.95, eps=1e-8, weight_decay=0.05, no_decay_modules=pats)
    for n, (idx, p, m, v) in want.items():
        l = leaves[n]
        sl = slice(l.offset, l.offset + l.numel)
        # 1e-6 of the leaf's scale: fp32 rounding of p itself; a decay applied to a masked leaf (or left
        # out of an unmasked one) moves an element by lr * wd * p * 2 = 1e-4 p
        assert (model.master[sl][idx].double().cpu() - p).abs().max().item() <= 1e-6 * p.abs().max().item(), n
        assert (model.m[sl][idx].double().cpu() - m).abs().max().item() <= 1e-6 * m.abs().max().item() + 1e-12, n
        assert (model.v[sl][idx].double().cpu() - v).abs().max().item() <= 1e-6 * v.abs().max().item() + 1e-20, n
        assert torch.equal(model.params_bf16[sl], model.master[sl].to(BF)), n
    # the tolerance does tell the two groups apart: the matrix against an oracle run WITHOUT decay misses
    n = "layers.3.mlp.down_proj.weight"
    idx, p, _, _ = want[n]
    l = leaves[n]
    p0 = before[n]
    g = G[n].reshape(-1)[idx].double().cpu()
    m, v = torch.zeros_like(p0), torch.zeros_like(p0)
    for step in (1, 2):
        p0, m, v = ref.adamw_step(p0, g, m, v, step=step, lr=1e-3, b1=0.9, b2=0.95, eps=1e-8, wd=0.0)
    assert (model.master[l.offset: l.offset + l.numel][idx].double().cpu() - p0).abs().max().item() > 1e-6 * p.abs().max().item()


def test_config3_llama7b_full_model():
    """The benchmark configuration itself: 32 layers, 7.3 B parameters, 8192 tokens."""
    say("config 3: Llama-like 7B, full model")
    from olmax_amd import TransformerRecipe
    cfg = TransformerRecipe.llama_like_7B_bench()
    model = cfg.build(batch_size=2, sequence_length=4096, seed=0)
    assert model.num_params == 7_298_355_200
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, cfg.vocab_size, (8192,), generator=g, dtype=torch.int32).cuda()
    labels = torch.randint(0, cfg.vocab_size, (8192,), generator=g, dtype=torch.int32).cuda()
    loss_ac = model.loss_and_grads(ids, labels).item()
    # N(0, 0.02) head on unit-RMS features: logits ~ N(0, 0.02^2 * 4096) -> loss = ln V + sigma^2 / 2
    want = math.log(cfg.vocab_size) + 0.5 * (0.02 ** 2) * 4096
    assert abs(loss_ac - want) < 0.05, (loss_ac, want)
    # checksum of the gradients with full-block recompute == without (same kernels, same order)
    chk = model.grad_bf16.float().abs().sum().item()
    first = model.grad_bf16[-4096:].clone()
    model.c.checkpoint = 0
    model._workspace = None
    torch.cuda.empty_cache()
    loss_keep = model.loss_and_grads(ids, labels).item()
    assert loss_keep == loss_ac
    assert model.grad_bf16.float().abs().sum().item() == chk
    assert torch.equal(model.grad_bf16[-4096:], first)
    # token index work is bit-exact: embedding rows of the first tokens
    emb = model.named_parameters()["embedding.weight"]
    ws_rows = model.workspace().view(torch.bfloat16)[: 4 * cfg.d_model].view(4, cfg.d_model)
    assert torch.equal(ws_rows, emb[ids[:4].long()].to(BF))

    # The step the benchmark times (second stream, full-block recompute, LM-head update cut into 32
    # pieces) against the sequential step, from the same seeded state: integer checksums of the
    # bit patterns of master / m / v / bf16 copy over the LM head and three layers must be equal
    # (AdamW is elementwise, the bf16 gradients are deterministic).
    from olmax_amd import _lib
    model.c.checkpoint = 1
    model._workspace = None
    torch.cuda.empty_cache()
    leaves = {model.leaf_name(l): l for l in model.leaves}
    spans = {"lm_head": (leaves["lm_head.proj.weight"].offset, leaves["lm_head.proj.weight"].numel)}
    for l in (0, 15, 31):
        first, last = leaves[f"layers.{l}.attention.q_proj.weight"], leaves[f"layers.{l}.mlp.down_proj.weight"]
        spans[f"layer{l}"] = (first.offset, last.offset + last.numel - first.offset)

    def checksums():
        out = {}
        for k, (o, n) in spans.items():
            out[k] = tuple(int(getattr(model, b)[o: o + n].view(torch.int32 if b != "params_bf16" else torch.int16)
                               .sum(dtype=torch.int64).item()) for b in ("master", "m", "v", "params_bf16"))
        return out

    kw = dict(step=1, lr=1e-4, b1=0.9, b2=0.95, weight_decay=0.1, no_decay_modules=["embedding.weight"])
    res = []
    for overlap in (False, True):
        model.reset_parameters(0)
        model.init_optimizer_state()
        loss = model.train_step(ids, labels, overlap_optimizer=overlap, **kw).item()
        n_launch = _lib.load().olmax_model_last_step_overlapped_launches()
        assert (n_launch >= 34 + 32) if overlap else n_launch == 0, n_launch  # 32 layers + norm + embedding, 32 head pieces
        torch.cuda.synchronize()
        res.append((loss, checksums()))
    assert res[0][0] == res[1][0] == loss_ac
    assert res[0][1] == res[1][1]


@pytest.mark.parametrize("name", ["llama3_8B", "olmo2_32B"])
def test_gqa_recipes_two_layer_slices_full_width(name):
    """Two-layer slices of the reference's grouped-query recipes at their real widths
    (src/olmax/nn/transformer/recipes.py:126-165 and :246-282): llama3-8B (32 query / 8 KV heads,
    SwiGLU 14336, vocab 128256) and OLMo2-32B (40 / 8 heads, d 5120, reordered norm + QK-norm,
    hidden 27648); causal-prefix parity against the oracle at seq 2048, micro-batch 2."""
    say(f"{name}: 2-layer slice at full width")
    from olmax_amd import TransformerRecipe
    hcfg = getattr(TransformerRecipe, name)()
    hcfg.num_layers = 2
    hcfg.norm_eps = 1e-6
    hcfg.layer_ac_policy = "nothing_saveable"
    ocfg = ref.ModelConfig(vocab=hcfg.vocab_size, d_model=hcfg.d_model, n_layers=2, n_heads=hcfg.n_heads,
                           n_kv_heads=hcfg.n_kv_heads, head_dim=128, hidden=hcfg.hidden_size,
                           layer_type="reordered" if hcfg.layer_type == "reordered_norm" else "pre",
                           qk_norm=bool(hcfg.qk_norm_headwise), eps=1e-6, rope_theta=hcfg.rope_theta)
    model, loss = _model_prefix_check(hcfg, ocfg, 2, 2048, seed=21)
    # unit-RMS hidden state times an N(0, 0.02) head: logits ~ N(0, d * 0.02^2), so the loss at
    # init is ln V + variance / 2
    assert abs(loss - (math.log(hcfg.vocab_size) + hcfg.d_model * 0.02 ** 2 / 2)) < 0.3
