"""GPU parity of the block / model / train-step entry points against the CPU oracle."""
import sys

import pytest
import torch

from oracle import ref

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
rt = ref.bf16_round


def say(msg):
    print(f"[case] {msg}", flush=True)


def cosine(a, b):
    a, b = a.double().cpu().flatten(), b.double().cpu().flatten()
    return (a @ b / (a.norm() * b.norm() + 1e-30)).item()


def relerr(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).norm() / (b.norm() + 1e-30)).item()


def _cfgs(kind, D=128, full_qk=False):
    """full_qk: QK-norm over the full projection width instead of per head (attention.py:281-284)."""
    from olmax_amd import TransformerConfig
    gem = kind == "gemma"
    H, K = (4, 2) if gem else (2, 2)
    ocfg = ref.ModelConfig(vocab=512, d_model=256, n_layers=2, n_heads=H, n_kv_heads=K, head_dim=D, hidden=512,
                           layer_type={"default": "pre", "reordered_norm": "reordered", "gemma": "gemma"}[kind],
                           act="gelu" if gem else "silu", qk_norm=kind != "default" or full_qk, qk_norm_headwise=not full_qk,
                           eps=1e-6, rope_theta=1e4,
                           rope_theta_layers=[1e4, 1e6] if gem else None, windows=[40, None] if gem else None,
                           attn_softcap=50.0 if gem else 0.0, final_softcap=30.0 if gem else 0.0, tied=gem)
    hcfg = TransformerConfig(vocab_size=512, d_model=256, hidden_size=512, num_layers=2, n_heads=H, n_kv_heads=K,
                             head_dim=D, layer_type=kind, activation="gelu" if gem else "silu",
                             qk_norm_headwise=kind != "default" and not full_qk, qk_norm=kind != "default" or full_qk,
                             norm_eps=1e-6, rope_theta=1e4,
                             rope_theta_per_layer=[1e4, 1e6] if gem else None,
                             window_size_per_layer=[40, None] if gem else None,
                             attn_logit_softcap=50.0 if gem else 0.0, final_logit_softcap=30.0 if gem else 0.0,
                             tie_embeddings=gem)
    return ocfg, hcfg


def _params(ocfg, seed=1):
    P = ref.init_params(ocfg, seed=seed)
    g = torch.Generator().manual_seed(seed + 100)
    out = {}
    for k, v in P.items():
        if "norm" in k:
            v = v + 0.1 * torch.randn(v.shape, generator=g)
        else:
            v = v * 2.0  # larger weights make every path matter
        out[k] = rt(v.float())
    return out


@pytest.mark.parametrize("kind,D,full_qk", [(k, D, False) for k in ("default", "reordered_norm", "gemma") for D in (128, 64)]
                         + [("default", 128, True), ("reordered_norm", 64, True), ("gemma", 128, True)])
def test_model_loss_and_grads_match_oracle(kind, D, full_qk):
    say(f"model grads kind={kind} D={D} full-width qk-norm={full_qk}")
    ocfg, hcfg = _cfgs(kind, D, full_qk)
    B, S = 2, 128
    P = _params(ocfg)
    gen = torch.Generator().manual_seed(5)
    ids = torch.randint(0, 512, (B, S), generator=gen, dtype=torch.int32)
    labels = torch.randint(0, 512, (B, S), generator=gen, dtype=torch.int32)
    labels[0, 3] = -100
    labels[1, 7] = 512  # the loader's label == V case
    model = hcfg.build(batch_size=B, sequence_length=S)
    model.load_state_dict(P)
    loss = model.loss_and_grads(ids.cuda().reshape(-1), labels.cuda().reshape(-1)).item()
    G = model.named_gradients()
    wloss, WG = ref.model_loss_and_grads(ocfg, {k: v.double() for k, v in P.items()}, ids, labels.long(), rt)
    assert abs(loss - wloss.item()) < 1e-2 * abs(wloss.item()), (loss, wloss.item())
    assert set(G) == set(WG)
    worst = min((cosine(G[n], WG[n]), n) for n in G)
    assert worst[0] >= 0.999, worst
    # forward-only entry point gives the same loss
    assert abs(model.forward_loss(ids.cuda().reshape(-1), labels.cuda().reshape(-1)).item() - loss) < 1e-6


def test_full_block_recompute_is_bitwise_identical():
    say("checkpoint == no checkpoint")
    ocfg, hcfg = _cfgs("default")
    B, S = 2, 128
    P = _params(ocfg)
    gen = torch.Generator().manual_seed(6)
    ids = torch.randint(0, 512, (B * S,), generator=gen, dtype=torch.int32).cuda()
    labels = torch.randint(0, 512, (B * S,), generator=gen, dtype=torch.int32).cuda()
    res = []
    for pol in (None, "nothing_saveable"):
        hcfg.layer_ac_policy = pol
        m = hcfg.build(batch_size=B, sequence_length=S)
        m.load_state_dict(P)
        l = m.loss_and_grads(ids, labels).item()
        res.append((l, m.grad_bf16.clone(), m.grad_f32.clone()))
    assert res[0][0] == res[1][0]
    assert torch.equal(res[0][1], res[1][1])
    # fp32 accumulators are filled by atomics (order varies): equal to rounding noise
    assert (res[0][2] - res[1][2]).abs().max() <= 1e-3 * res[0][2].abs().max()


def test_tiny_llama_ten_train_steps_follow_oracle():
    """BASELINE config 1 (4 layers, d 256, 4x64 heads, hidden 1024, vocab 4096, seq 512, mb 4,
    AdamW lr 3e-4 betas .9/.95 wd .1): the loss curve of the HIP path follows the CPU oracle."""
    say("tiny llama 10 steps")
    from olmax_amd import AdamWConfig, ConstantSchedule, Trainer, TransformerRecipe
    hcfg = TransformerRecipe.tiny_llama()
    ocfg = ref.ModelConfig(vocab=4096, d_model=256, n_layers=4, n_heads=4, n_kv_heads=4, head_dim=64, hidden=1024,
                           eps=1e-6, rope_theta=1e4)
    B, S = 4, 512
    master = ref.init_params(ocfg, seed=0)
    model = hcfg.build(batch_size=B, sequence_length=S)
    model.load_state_dict(master)
    tr = Trainer(model, AdamWConfig(lr=ConstantSchedule(3e-4), b1=0.9, b2=0.95, weight_decay=0.1))
    opt = {"m": {k: torch.zeros_like(v) for k, v in master.items()}, "v": {k: torch.zeros_like(v) for k, v in master.items()}}
    got, want = [], []
    for step in range(1, 11):
        gen = torch.Generator().manual_seed(step)
        ids = torch.randint(0, 4096, (B, S), generator=gen, dtype=torch.int32)
        labels = torch.randint(0, 4096, (B, S), generator=torch.Generator().manual_seed(step + 1000), dtype=torch.int32)
        got.append(tr.process_microbatch(ids.cuda().reshape(-1), labels.cuda().reshape(-1)).item())
        want.append(ref.train_step(ocfg, master, opt, ids, labels.long(), step=step, lr=3e-4, b1=0.9, b2=0.95, wd=0.1,
                                   no_decay=(), compute_bf16=True)[0].item())
    print("hip   :", [round(x, 4) for x in got]); print("oracle:", [round(x, 4) for x in want], flush=True)
    for a, b in zip(got, want):
        assert abs(a - b) < 1e-2 * abs(b)
    # parameters after 10 steps agree
    for n, p in model.named_parameters().items():
        assert relerr(p, master[n]) < 1e-2, n  # early Adam steps are ~lr*sign(g): tiny grads flip


def test_grad_clipping_and_embedding_decay_mask():
    say("clip + decay mask")
    from olmax_amd import AdamWConfig, ConstantSchedule, Trainer
    ocfg, hcfg = _cfgs("default")
    B, S = 1, 128
    model = hcfg.build(batch_size=B, sequence_length=S)
    P = _params(ocfg)
    model.load_state_dict(P)
    tr = Trainer(model, AdamWConfig(lr=ConstantSchedule(1e-3), weight_decay=0.5, no_decay_modules=["embedding.weight"],
                                    max_grad_norm=0.05))
    gen = torch.Generator().manual_seed(2)
    ids = torch.randint(0, 512, (B * S,), generator=gen, dtype=torch.int32).cuda()
    before = {k: v.clone() for k, v in model.named_parameters().items()}
    tr.process_microbatch(ids, ids)
    G = model.named_gradients()
    gnorm = sum((g.double() ** 2).sum().item() for g in G.values()) ** 0.5
    assert abs(tr.grad_norm - gnorm) < 1e-3 * gnorm
    # rows of the embedding that received no gradient: masked from decay -> unchanged
    unused = torch.ones(512, dtype=torch.bool); unused[ids.cpu().long()] = False
    emb = model.named_parameters()["embedding.weight"]
    assert torch.equal(emb[unused.cuda()], before["embedding.weight"][unused.cuda()])
    # an ordinary matrix does decay
    assert not torch.equal(model.named_parameters()["layers.0.mlp.up_proj.weight"], before["layers.0.mlp.up_proj.weight"])


def test_weight_decay_mask_takes_any_fnmatch_pattern():
    """no_decay_modules are fnmatch patterns over the leaf paths (src/olmax/optim/config.py:94-122).
    With all gradients zero AdamW is pure decay: a masked leaf must not move at all, every other
    leaf becomes p (1 - lr wd); through the whole-model AdamW, the accumulated-gradient AdamW and
    the overlapped train step (there against the sequential one, with real gradients)."""
    say("weight-decay mask by pattern")
    from olmax_amd import AdamWConfig, ConstantSchedule, Trainer
    import fnmatch
    ocfg, hcfg = _cfgs("gemma")
    B, S = 1, 128
    pats = ["embedding.weight", "*norm.weight", "layers.1.mlp.up_proj.weight"]
    P = _params(ocfg)
    for path in ("adamw", "accumulated"):
        model = hcfg.build(batch_size=B, sequence_length=S)
        model.load_state_dict(P)
        before = {k: v.clone() for k, v in model.named_parameters().items()}
        model.grad_bf16.zero_(); model.grad_f32.zero_()
        if path == "adamw":
            model.adamw_step(step=1, lr=0.1, weight_decay=0.25, no_decay_modules=pats)
        else:
            model.accumulate_grads(0)
            model.adamw_step_accumulated(step=1, lr=0.1, weight_decay=0.25, no_decay_modules=pats)
        n_masked = 0
        for n, p in model.named_parameters().items():
            masked = any(fnmatch.fnmatch(n, pat) for pat in pats)
            n_masked += masked
            want = before[n] if masked else before[n] * (1 - 0.1 * 0.25)
            assert (p - want).abs().max().item() <= (0 if masked else 1e-7), (path, n)
        assert n_masked == 1 + 2 * 6 + 1 + 1  # embedding, six norm weights per gemma layer with QK-norm, final norm, one matrix
        assert torch.equal(model.params_bf16, model.master.to(BF))  # the bf16 working copy follows the master copy
    with pytest.warns(UserWarning, match="did not match"):
        model.weight_decay_mask(["no.such.leaf"])
    # the same update with lr and the bias corrections read from device memory (step / lr arguments ignored)
    m1 = hcfg.build(batch_size=B, sequence_length=S); m1.load_state_dict(P)
    m2 = hcfg.build(batch_size=B, sequence_length=S); m2.load_state_dict(P)
    for mm in (m1, m2):
        mm.grad_bf16.normal_(0, 0.01, generator=torch.Generator(device="cuda").manual_seed(1)); mm.grad_f32.fill_(0.01)
    m1.adamw_step(step=3, lr=0.02, b1=0.9, b2=0.95, weight_decay=0.25, no_decay_modules=pats)
    f = lambda x: float(torch.tensor(x, dtype=torch.float32))  # b1 / b2 reach the library as fp32
    hyper = torch.tensor([0.02, 1 - f(0.9) ** 3, 1 - f(0.95) ** 3], dtype=torch.float64).float().cuda()
    m2.adamw_step(step=0, lr=0.0, b1=0.9, b2=0.95, weight_decay=0.25, no_decay_modules=pats, hyper_dev=hyper)
    assert torch.equal(m1.master, m2.master) and torch.equal(m1.params_bf16, m2.params_bf16)
    # overlapped (per-layer AdamW on a second stream) == sequential, with the same mask and real gradients
    hcfg.layer_ac_policy = "nothing_saveable"
    gen = torch.Generator().manual_seed(4)
    ids = torch.randint(0, 512, (B * S,), generator=gen, dtype=torch.int32).cuda()
    outs = []
    for overlap in (False, True):
        model = hcfg.build(batch_size=B, sequence_length=S)
        model.load_state_dict(P)
        tr = Trainer(model, AdamWConfig(lr=ConstantSchedule(1e-2), weight_decay=0.5, no_decay_modules=pats), overlap_optimizer=overlap)
        tr.process_microbatch(ids, ids)
        torch.cuda.synchronize()
        outs.append(model.master.clone())
    assert relerr(outs[1], outs[0]) < 1e-5


@pytest.mark.parametrize("kind,full_qk", [("reordered_norm", False), ("default", False), ("gemma", False), ("reordered_norm", True)])
def test_single_block_fwd_bwd(kind, full_qk):
    """BASELINE config 2 at reduced width: one block forward+backward in isolation."""
    say(f"single block {kind} full-width qk-norm={full_qk}")
    from olmax_amd.layer import TransformerBlock
    ocfg, hcfg = _cfgs(kind, full_qk=full_qk)
    ocfg.n_layers = hcfg.num_layers = 1
    if kind == "gemma":
        ocfg.windows, ocfg.rope_theta_layers = [40], [1e4]
        hcfg.window_size_per_layer, hcfg.rope_theta_per_layer = [40], [1e4]
    B, S, d = 2, 128, 256
    P = {k.replace("layers.0.", ""): v for k, v in _params(ocfg).items() if k.startswith("layers.0.")}
    blk = TransformerBlock(hcfg, batch_size=B, sequence_length=S)
    blk.load_state_dict(P)
    gen = torch.Generator().manual_seed(9)
    x = torch.randn(B, S, d, generator=gen).to(BF); dy = torch.randn(B, S, d, generator=gen).to(BF)
    y = blk.forward(x.cuda().reshape(B * S, d))
    dx = blk.backward(dy.cuda().reshape(B * S, d))
    Pd = {"layers.0." + k: v.double() for k, v in P.items()}
    wy, tape = ref.block_fwd(ocfg, Pd, 0, x.double(), rt)
    G = {}
    wdx = ref.block_bwd(ocfg, Pd, 0, dy.double(), tape, G, rt)
    assert relerr(y, wy.reshape(B * S, d)) < 1e-2
    assert cosine(dx, wdx) >= 0.999
    for n, g in blk.grads.items():
        assert cosine(g, G["layers.0." + n]) >= 0.999, n


def _overlapped_launches():
    from olmax_amd import _lib
    return _lib.load().olmax_model_last_step_overlapped_launches()


def test_overlapped_optimizer_equals_sequential():
    """AdamW launched per layer on a second stream during the backward pass gives the same
    parameters as loss_and_grads followed by the whole-model AdamW.  The overlapped branch only
    exists with full-block recompute; the library's launch counter proves which branch ran."""
    say("overlapped optimizer == sequential")
    from olmax_amd import AdamWConfig, ConstantSchedule, Trainer
    ocfg, hcfg = _cfgs("gemma")
    hcfg.layer_ac_policy = "nothing_saveable"
    B, S = 2, 128
    P = _params(ocfg)
    outs = []
    for overlap in (False, True):
        model = hcfg.build(batch_size=B, sequence_length=S)
        model.load_state_dict(P)
        tr = Trainer(model, AdamWConfig(lr=ConstantSchedule(1e-3), weight_decay=0.1), overlap_optimizer=overlap)
        losses = []
        for step in range(3):
            gen = torch.Generator().manual_seed(step)
            ids = torch.randint(0, 512, (B * S,), generator=gen, dtype=torch.int32).cuda()
            labels = torch.randint(0, 512, (B * S,), generator=gen, dtype=torch.int32).cuda()
            losses.append(tr.process_microbatch(ids, labels).item())
            # final norm, one group per layer, the embedding
            assert _overlapped_launches() == (hcfg.num_layers + 2 if overlap else 0)
        torch.cuda.synchronize()
        outs.append((losses, model.master.clone(), model.params_bf16.clone()))
    assert outs[0][0] == pytest.approx(outs[1][0], rel=1e-5)
    assert relerr(outs[1][1], outs[0][1]) < 1e-5
    assert (outs[0][2].float() - outs[1][2].float()).abs().max() <= 1e-2 * outs[0][2].float().abs().max()


def _untied_llama(n_layers=4, vocab=4112):
    """An untied Llama-type model whose LM head (vocab x 256) is larger than one layer (655 872
    parameters), so that the overlapped step cuts the head's update into a layer-sized first piece,
    even shares that are not multiples of 8 elements (vocab 4112, 4 layers: 132 268) and a clipped
    last one.  Head dim 128: every bf16 gradient comes from deterministic kernels."""
    from olmax_amd import TransformerConfig
    ocfg = ref.ModelConfig(vocab=vocab, d_model=256, n_layers=n_layers, n_heads=2, n_kv_heads=2, head_dim=128, hidden=512,
                           eps=1e-6, rope_theta=1e4)
    hcfg = TransformerConfig(vocab_size=vocab, d_model=256, hidden_size=512, num_layers=n_layers, n_heads=2, head_dim=128,
                             norm_eps=1e-6, rope_theta=1e4, layer_ac_policy="nothing_saveable")
    return ocfg, hcfg


@pytest.mark.parametrize("n_layers,vocab", [(4, 4112), (3, 8200), (5, 2056)])
def test_overlapped_step_on_an_untied_model_is_bit_equal_to_the_sequential_step(n_layers, vocab):
    """The measured path: olmax_model_train_step with a second stream, full-block recompute and an
    UNTIED model, whose LM-head update is spread in pieces over the layers' recompute windows.
    AdamW is elementwise and the bf16 gradients are deterministic, so from the same state both
    orders must leave master, m, v and the bf16 working copy of every bf16-gradient leaf BIT-equal
    (a skipped, doubled or misaligned range of the head cannot hide); leaves whose gradients are
    summed by fp32 atomics (embedding, norm weights) agree to rounding noise.  Three consecutive
    steps (non-zero moments, step counts 1-3), each started from the sequential run's state.
    (vocab 2056: head smaller than a layer, one piece; 8200 x 3 layers: head of 3.2 layers.)"""
    say(f"overlapped untied train step, bitwise, layers={n_layers} vocab={vocab}")
    ocfg, hcfg = _untied_llama(n_layers, vocab)
    B, S = 2, 128
    P = _params(ocfg)
    seq = hcfg.build(batch_size=B, sequence_length=S); seq.load_state_dict(P)
    ovl = hcfg.build(batch_size=B, sequence_length=S); ovl.load_state_dict(P)
    for mdl in (seq, ovl):
        mdl.init_optimizer_state()
    kw = dict(lr=1e-3, b1=0.9, b2=0.95, weight_decay=0.1, no_decay_modules=["embedding.weight"])
    for step in range(1, 4):
        gen = torch.Generator().manual_seed(40 + step)
        ids = torch.randint(0, vocab, (B * S,), generator=gen, dtype=torch.int32).cuda()
        labels = torch.randint(0, vocab, (B * S,), generator=gen, dtype=torch.int32).cuda()
        for name in ("master", "m", "v", "params_bf16"):
            getattr(ovl, name).copy_(getattr(seq, name))
        l0 = seq.train_step(ids, labels, step=step, overlap_optimizer=False, **kw).item()
        assert _overlapped_launches() == 0
        l1 = ovl.train_step(ids, labels, step=step, overlap_optimizer=True, **kw).item()
        n_launch = _overlapped_launches()
        assert n_launch >= n_layers + 2, n_launch  # layers, final norm (+ head pieces), embedding
        torch.cuda.synchronize()
        assert l0 == l1
        assert torch.equal(seq.grad_bf16, ovl.grad_bf16)
        for leaf in seq.leaves:
            sl = slice(leaf.offset, leaf.offset + leaf.numel)
            name = seq.leaf_name(leaf)
            for buf in ("master", "m", "v", "params_bf16"):
                a, b = getattr(seq, buf)[sl], getattr(ovl, buf)[sl]
                if not leaf.grad_f32:
                    assert torch.equal(a, b), (step, name, buf, (a.float() - b.float()).abs().max().item())
                else:
                    assert (a.float() - b.float()).abs().max().item() <= 1e-5 * a.float().abs().max().item() + 1e-12, (step, name, buf)
        # every element of the head moved (Adam's first steps are ~lr in size wherever g != 0)
        head = next(l for l in seq.leaves if seq.leaf_name(l) == "lm_head.proj.weight")
        if step == 1:
            moved = ovl.master[head.offset: head.offset + head.numel] != P["lm_head.proj.weight"].cuda().reshape(-1)
            assert moved.float().mean().item() > 0.999


def test_overlapped_untied_ten_steps_follow_oracle():
    """The same untied, checkpointed, overlapped configuration driven through Trainer for 10 steps
    against the oracle's train_step (bf16 compute): loss curve and final parameters."""
    say("overlapped untied llama 10 steps vs oracle")
    from olmax_amd import AdamWConfig, ConstantSchedule, Trainer
    ocfg, hcfg = _untied_llama(4, 4112)
    B, S = 2, 128
    master = ref.init_params(ocfg, seed=2)
    model = hcfg.build(batch_size=B, sequence_length=S)
    model.load_state_dict(master)
    tr = Trainer(model, AdamWConfig(lr=ConstantSchedule(3e-4), b1=0.9, b2=0.95, weight_decay=0.1), overlap_optimizer=True)
    opt = {"m": {k: torch.zeros_like(v) for k, v in master.items()}, "v": {k: torch.zeros_like(v) for k, v in master.items()}}
    got, want = [], []
    for step in range(1, 11):
        gen = torch.Generator().manual_seed(70 + step)
        ids = torch.randint(0, 4112, (B, S), generator=gen, dtype=torch.int32)
        labels = torch.randint(0, 4112, (B, S), generator=gen, dtype=torch.int32)
        got.append(tr.process_microbatch(ids.cuda().reshape(-1), labels.cuda().reshape(-1)).item())
        assert _overlapped_launches() > 0
        want.append(ref.train_step(ocfg, master, opt, ids, labels.long(), step=step, lr=3e-4, b1=0.9, b2=0.95, wd=0.1,
                                   no_decay=(), compute_bf16=True)[0].item())
    print("hip   :", [round(x, 4) for x in got]); print("oracle:", [round(x, 4) for x in want], flush=True)
    for a, b in zip(got, want):
        assert abs(a - b) < 1e-2 * abs(b)
    for n, p in model.named_parameters().items():
        assert relerr(p, master[n]) < 1e-2, n
    assert torch.equal(model.params_bf16, model.master.to(BF))


def test_train_batch_gradient_accumulation_follows_oracle_and_mean_identity():
    """train_batch with k micro-batches (optax.MultiSteps semantics: running fp32 mean of the
    gradients, one clipped AdamW step per batch, loss = mean of micro-batch losses) against the
    oracle on the tiny Llama, plus two properties that need no oracle: k copies of one micro-batch
    equal a single step on it, and the accumulator equals the plain mean of the gradients."""
    say("train_batch / gradient accumulation")
    from olmax_amd import AdamWConfig, ConstantSchedule, Trainer, TransformerRecipe
    hcfg = TransformerRecipe.tiny_llama()
    ocfg = ref.ModelConfig(vocab=4096, d_model=256, n_layers=4, n_heads=4, n_kv_heads=4, head_dim=64, hidden=1024,
                           eps=1e-6, rope_theta=1e4)
    B, S, K = 2, 256, 3
    master = ref.init_params(ocfg, seed=0)
    init = {k: v.clone() for k, v in master.items()}

    def batch_of(step):
        out = []
        for j in range(K):
            gen = torch.Generator().manual_seed(100 * step + j)
            ids = torch.randint(0, 4096, (B, S), generator=gen, dtype=torch.int32)
            labels = torch.randint(0, 4096, (B, S), generator=gen, dtype=torch.int32)
            out.append((ids, labels))
        return out

    opt_cfg = AdamWConfig(lr=ConstantSchedule(3e-4), b1=0.9, b2=0.95, weight_decay=0.1, max_grad_norm=1.0)
    model = hcfg.build(batch_size=B, sequence_length=S)
    model.load_state_dict(master)
    tr = Trainer(model, opt_cfg)
    opt = {"m": {k: torch.zeros_like(v) for k, v in master.items()}, "v": {k: torch.zeros_like(v) for k, v in master.items()}}
    for step in range(1, 4):
        batch = batch_of(step)
        got = tr.train_batch([(i.cuda().reshape(-1), l.cuda().reshape(-1)) for i, l in batch]).item()
        want, acc = ref.train_batch(ocfg, master, opt, [(i, l.long()) for i, l in batch], step=step, lr=3e-4, b1=0.9, b2=0.95,
                                    wd=0.1, no_decay=(), compute_bf16=True, max_grad_norm=1.0)
        assert abs(got - float(want)) < 1e-2 * abs(float(want))
        assert tr.count == step
    for n, p in model.named_parameters().items():
        assert relerr(p, master[n]) < 1e-2, n
    # the accumulator of the last batch is the clipped mean in the oracle; compare directions
    leaves = {model.leaf_name(l): l for l in model.leaves}
    for n in ("layers.1.mlp.down_proj.weight", "embedding.weight", "layers.0.attention_norm.weight"):
        l = leaves[n]
        assert cosine(model.grad_acc[l.offset: l.offset + l.numel].view(acc[n].shape), acc[n]) >= 0.999, n

    # mean identity: accumulate three different gradients, compare with their plain mean
    model2 = hcfg.build(batch_size=B, sequence_length=S)
    model2.load_state_dict(init)
    gs = []
    for j, (ids, labels) in enumerate(batch_of(9)):
        model2.loss_and_grads(ids.cuda().reshape(-1), labels.cuda().reshape(-1))
        model2.accumulate_grads(j)
        gs.append(model2.grad_bf16.float().clone())
    l = leaves["layers.2.attention.q_proj.weight"]
    sl = slice(l.offset, l.offset + l.numel)
    mean = (gs[0][sl] + gs[1][sl] + gs[2][sl]) / 3
    assert (model2.grad_acc[sl] - mean).abs().max() <= 1e-6 * mean.abs().max() + 1e-12

    # k copies of one micro-batch == one step on it (no clipping, so the paths differ only in
    # where the bf16 gradient is widened)
    one = batch_of(5)[0]
    dev = (one[0].cuda().reshape(-1), one[1].cuda().reshape(-1))
    res = []
    for k in (1, 2):
        m = hcfg.build(batch_size=B, sequence_length=S)
        m.load_state_dict(init)
        t = Trainer(m, AdamWConfig(lr=ConstantSchedule(3e-4), b1=0.9, b2=0.95, weight_decay=0.1), overlap_optimizer=False)
        t.train_batch([dev] * k)
        res.append(m.master.clone())
    # (a first Adam step is ~lr*sign(g): gradients summed by atomics in another order may flip
    # near-zero entries, worth at most lr = 3e-4 against parameters of scale 0.02-0.1)
    assert relerr(res[1], res[0]) < 5e-3


def test_checkpoint_round_trip_resumes_the_run(tmp_path):
    """save_checkpoint / load_checkpoint (TrainState of src/olmax/train/trainer.py:45-53): a run
    resumed from the file continues like the uninterrupted one, including the data loader
    position: the first resumed loss is bit-identical (same parameters, deterministic forward),
    later ones agree to the noise of the atomically summed norm / embedding gradients (which an
    early Adam step, ~lr*sign(g), amplifies).  Profiler ranges are switched on for the run."""
    say("checkpoint round trip")
    from olmax_amd import AdamWConfig, Trainer, TransformerRecipe, WarmupCosineDecaySchedule, data
    hcfg = TransformerRecipe.tiny_llama()
    B, S = 2, 128
    ocfg = ref.ModelConfig(vocab=4096, d_model=256, n_layers=4, n_heads=4, n_kv_heads=4, head_dim=64, hidden=1024,
                           eps=1e-6, rope_theta=1e4)
    P = ref.init_params(ocfg, seed=3)
    sched = WarmupCosineDecaySchedule(2, 6, 1e-3, 1e-5, 1e-5)
    kw = dict(vocab_size=4096, sequence_length=S, global_batch_size_instances=B, total_batches=6)

    def fresh():
        m = hcfg.build(batch_size=B, sequence_length=S)
        m.load_state_dict(P)
        return Trainer(m, AdamWConfig(lr=sched, weight_decay=0.1, max_grad_norm=1.0), overlap_optimizer=False)

    Trainer.set_profiler_ranges(True)
    try:
        tr, dl = fresh(), data.DataLoader(11, **kw)
        losses = []
        path = str(tmp_path / "state.safetensors")
        for i, batch in enumerate(dl):
            losses.append(tr.train_batch([(x.reshape(-1), y.reshape(-1)) for x, y in batch]).item())
            if i == 2:
                tr.save_checkpoint(path, data_loader=dl, tokens_seen=3 * B * S)
        final = tr.model.master.clone()

        tr2, dl2 = fresh(), data.DataLoader(0, **kw)
        meta = tr2.load_checkpoint(path, data_loader=dl2)
        assert meta["step"] == 3 and meta["tokens_seen"] == 3 * B * S and tuple(meta["data_loader_state"]) == (11, 3, 0)
        assert tr2.count == 3 and dl2.get_state() == (11, 3, 0)
        resumed = [tr2.train_batch([(x.reshape(-1), y.reshape(-1)) for x, y in batch]).item() for batch in dl2]
    finally:
        Trainer.set_profiler_ranges(False)
    assert len(resumed) == 3
    assert resumed[0] == losses[3]
    assert resumed == pytest.approx(losses[3:], rel=1e-3)
    assert relerr(tr2.model.master, final) < 2e-2
    with pytest.raises(ValueError):
        small = TransformerRecipe.tiny_llama()
        small.num_layers = 2
        Trainer(small.build(batch_size=B, sequence_length=S), AdamWConfig(lr=sched)).load_checkpoint(path)


def test_fit_loop_logs_every_step_once_with_losses_of_a_manual_run():
    """Trainer.fit (training loop of src/olmax/train/trainer.py:531-637): every step is logged exactly
    once and in order, one step late; the logged losses, learning rates and gradient norms are those
    of the same run driven by hand; throughput follows TPS = BPS x tokens with the averages from the
    10th step on."""
    say("fit loop")
    from olmax_amd import AdamWConfig, Trainer, TransformerRecipe, WarmupCosineDecaySchedule, data
    hcfg = TransformerRecipe.tiny_llama()
    B, S, steps = 2, 128, 12
    ocfg = ref.ModelConfig(vocab=4096, d_model=256, n_layers=4, n_heads=4, n_kv_heads=4, head_dim=64, hidden=1024,
                           eps=1e-6, rope_theta=1e4)
    P = ref.init_params(ocfg, seed=5)
    sched = WarmupCosineDecaySchedule(3, 9, 1e-3, 1e-5, 1e-5)
    kw = dict(vocab_size=4096, sequence_length=S, global_batch_size_instances=2 * B, total_batches=steps + 3, num_microbatches=2)

    def fresh():
        m = hcfg.build(batch_size=B, sequence_length=S)
        m.load_state_dict(P)
        return Trainer(m, AdamWConfig(lr=sched, weight_decay=0.1, max_grad_norm=1.0), overlap_optimizer=False)

    tr = fresh()
    want = []
    for i, batch in enumerate(data.DataLoader(3, **kw)):
        if i == steps:
            break
        lr = tr.optim.lr_at(tr.count)
        loss = tr.train_batch([(x.reshape(-1), y.reshape(-1)) for x, y in batch]).item()
        want.append((loss, lr, tr.grad_norm))

    tr2 = fresh()
    logged = []
    dl2 = data.DataLoader(3, **kw)
    tr2.fit(dl2, max_steps=steps, log_fn=lambda s, m: logged.append((s, m)))
    assert dl2.get_state()[1] == steps  # the loader is not one batch ahead of what was trained on
    assert tr2.count == steps and [s for s, _ in logged] == list(range(1, steps + 1))
    for (s, m), (loss, lr, gn) in zip(logged, want):
        assert m["optim/lr"] == pytest.approx(lr, rel=1e-6)
        assert m["train/loss"] == pytest.approx(loss, rel=1e-3 if s > 1 else 1e-6)
        assert m["optim/g_norm"] == pytest.approx(gn, rel=2e-2)
        assert m["throughput/TPS"] == pytest.approx(m["throughput/BPS"] * 2 * B * S)
        assert ("throughput/TPS average" in m) == (s >= 10)


@pytest.mark.parametrize("overlap", [False, True])
def test_train_step_captured_in_a_hip_graph_replays_like_eager_steps(overlap):
    """The library only enqueues on the streams it is handed (zeroing is a fill kernel, the
    optimizer stream is forked and joined with events inside the call), so one train step can be
    recorded into a HIP graph once and replayed: with the token buffers and the three
    step-dependent scalars {lr, 1 - b1^t, 1 - b2^t} updated in place between replays, four
    replays must walk the same losses and parameters as four eager calls.  Every replay is
    checked, with eager copies and a synchronisation between replays."""
    say(f"train step under graph capture, overlap={overlap}")
    ocfg, hcfg = _cfgs("gemma")
    hcfg.layer_ac_policy = "nothing_saveable"
    B, S, steps = 2, 128, 5
    P = _params(ocfg)
    b1, b2 = 0.9, 0.95
    f = lambda x: float(torch.tensor(x, dtype=torch.float32))
    batches, hypers = [], []
    for t in range(1, steps + 1):
        gen = torch.Generator().manual_seed(100 + t)
        batches.append((torch.randint(0, 512, (B * S,), generator=gen, dtype=torch.int32).cuda(),
                        torch.randint(0, 512, (B * S,), generator=gen, dtype=torch.int32).cuda()))
        lr = 1e-3 * t  # a schedule that moves every step
        hypers.append(torch.tensor([lr, 1 - f(b1) ** t, 1 - f(b2) ** t], dtype=torch.float64).float().cuda())
    kw = dict(step=0, lr=0.0, b1=b1, b2=b2, weight_decay=0.1, overlap_optimizer=overlap)

    eager = hcfg.build(batch_size=B, sequence_length=S); eager.load_state_dict(P)
    want = []
    for (ids, labels), hy in zip(batches, hypers):
        loss = eager.train_step(ids, labels, hyper_dev=hy, **kw)
        want.append((loss.item(), eager.master.clone()))

    model = hcfg.build(batch_size=B, sequence_length=S); model.load_state_dict(P)
    ids_buf, labels_buf, hyper_buf = batches[0][0].clone(), batches[0][1].clone(), hypers[0].clone()
    # step 1 eagerly (kernel attributes, workspace and optimizer state exist before the capture starts)
    loss = model.train_step(ids_buf, labels_buf, hyper_dev=hyper_buf, **kw)
    assert loss.item() == pytest.approx(want[0][0], rel=1e-5)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        model.train_step(ids_buf, labels_buf, hyper_dev=hyper_buf, **kw)
    assert relerr(model.master, want[0][1]) < 1e-6  # recording ran nothing
    for t in range(1, steps):
        ids_buf.copy_(batches[t][0]); labels_buf.copy_(batches[t][1]); hyper_buf.copy_(hypers[t])
        graph.replay()
        torch.cuda.synchronize()
        assert model.loss.item() == pytest.approx(want[t][0], rel=1e-5), t
        assert relerr(model.master, want[t][1]) < 1e-5, t
        assert torch.equal(model.params_bf16, model.master.to(BF)), t
