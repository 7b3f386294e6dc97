#!/usr/bin/env python3
"""Benchmark of the HIP train step: Llama-like 7B, seq 4096, micro-batch 2, bf16 compute,
fp32 master weights + AdamW, full-block activation checkpointing, one MI355X.

Prints ONE JSON line: whole-job train tokens/s (inputs resident in HBM), bf16 MFU, the
roofline figures of the dominant kernel (the bf16 MFMA GEMM, timed live with HIP events on
its launch stream) and a CPU baseline (the CPU oracle, "port") on a bounded sample.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16 = 2.5e15  # dense MFMA bf16 FLOP/s of one MI355X
TRAFFIC_PROFILE = os.path.join("profiles", "gemm_traffic_pmc_llama7b_shapes.txt")


def gemm_traffic_bytes():
    """HBM-side bytes per launch (fetch + write) of the GEMM instantiations, keyed like
    olmax_gemm_profile_end, read from the `# traffic_bytes key=<k> bytes=<b>` lines of the committed
    rocprofv3 --pmc summary (FETCH_SIZE / WRITE_SIZE runs of this script, calibrated against a cast
    kernel of known size; the file gives the commands).  Counter runs are separate from the timed run:
    the figure describes the kernels of the build the summary was made from."""
    import re

    out = {}
    try:
        with open(os.path.join(ROOT, TRAFFIC_PROFILE)) as f:
            for line in f:
                m = re.match(r"#\s*traffic_bytes\s+key=(\d+)\s+bytes=([0-9.eE+]+)", line)
                if m:
                    out[int(m.group(1))] = float(m.group(2))
    except OSError:
        pass
    return out


def cpu_baseline(steps: int = 10):
    """The CPU oracle ("port" of the reference's JAX path) timed on this box's host cores.

    `value` is like for like with the headline metric: a BOUNDED sample of the same workload (one
    of the 32 blocks forward + backward + AdamW and the LM head + cross entropy of the 7B model on
    512 tokens of one sequence, fp32), scaled to tokens/s of the whole step as
    tokens / (32 x block + head).  Beside it, under `tiny_config`, the reference's own CPU-sized
    case (BASELINE configs[0]: 4 layers, d_model 256, 4 heads x 64, SwiGLU 1024, vocab 4096, seq
    512, micro-batch 4, fp32, AdamW lr 3e-4 betas 0.9/0.95 wd 0.1) run for real: `steps` full
    train steps, the first excluded, with the loss curve the HIP path is tested against."""
    import torch
    from oracle import ref

    threads = torch.get_num_threads()
    # ---- the headline workload, sampled
    cfg7 = ref.ModelConfig(vocab=100352, d_model=4096, n_layers=1, n_heads=32, n_kv_heads=32, head_dim=128,
                           hidden=11008, eps=1e-6, rope_theta=5e5)
    g = torch.Generator().manual_seed(0)
    P = {k: v for k, v in ref.init_params(cfg7, seed=0).items() if k.startswith("layers.0.")}
    n7 = 512
    x = torch.randn(1, n7, 4096, generator=g)
    dy = torch.randn(1, n7, 4096, generator=g)
    G = {}
    ref.block_fwd(cfg7, P, 0, x[:, :64])  # untimed warm-up of the thread pool and allocator
    t0 = time.perf_counter()
    y, tape = ref.block_fwd(cfg7, P, 0, x)
    ref.block_bwd(cfg7, P, 0, dy, tape, G)
    for n in P:
        ref.adamw_step(P[n], G[n], torch.zeros_like(P[n]), torch.zeros_like(P[n]), step=1, lr=1e-4)
    t_block = time.perf_counter() - t0
    W = torch.randn(100352, 4096, generator=g) * 0.02
    labels = torch.randint(0, 100352, (n7,), generator=g)
    t0 = time.perf_counter()
    ref.lm_head_ce(x[0], W, labels)
    t_head = time.perf_counter() - t0
    del P, G, W, tape
    out = {
        "value": n7 / (32 * t_block + t_head), "unit": "tokens/s", "cores": threads, "kind": "port",
        "sample": f"bounded sample of the headline workload (Llama-like 7B, fp32 torch-CPU oracle): 1 of 32 blocks fwd+bwd+AdamW "
                  f"({t_block:.2f} s) + LM head / cross entropy ({t_head:.2f} s) on {n7} tokens of one sequence, scaled as "
                  f"{n7} / (32 x block + head); no recompute, attention over {n7} keys instead of 4096 (which flatters the CPU)",
        "os_cpu_count": os.cpu_count(), "torch_threads": threads,
    }
    # ---- the reference's own CPU-sized case, run in full
    cfg = ref.ModelConfig(vocab=4096, d_model=256, n_layers=4, n_heads=4, n_kv_heads=4, head_dim=64, hidden=1024,
                          eps=1e-6, rope_theta=1e4)
    B, S = 4, 512
    master = ref.init_params(cfg, seed=0)
    opt = {"m": {k: torch.zeros_like(v) for k, v in master.items()}, "v": {k: torch.zeros_like(v) for k, v in master.items()}}
    times, losses = [], []
    for step in range(1, steps + 1):
        gen = torch.Generator().manual_seed(step - 1)
        ids = torch.randint(0, 4096, (B, S), generator=gen, dtype=torch.int32)
        labels = torch.randint(0, 4096, (B, S), generator=torch.Generator().manual_seed(step), dtype=torch.int64)
        t0 = time.perf_counter()
        loss, _ = ref.train_step(cfg, master, opt, ids, labels, step=step, lr=3e-4, b1=0.9, b2=0.95, wd=0.1, no_decay=())
        times.append(time.perf_counter() - t0)
        losses.append(round(float(loss), 5))
    timed = times[1:] if len(times) > 1 else times
    tok = B * S
    out["tiny_config"] = {
        "value": tok * len(timed) / sum(timed), "unit": "tokens/s", "tokens_per_s_best_step": tok / min(timed),
        "note": f"a DIFFERENT, CPU-sized workload (BASELINE configs[0]: tiny Llama, 4 layers, d 256, vocab 4096, seq 512, micro-batch 4, "
                f"fp32 + AdamW): {steps} full train steps of the oracle, first step excluded ({sum(timed):.2f} s timed); not comparable "
                f"with the headline value",
        "loss_curve": losses}
    return out


def hbm_kernels(T: int, d: int, F: int, heads: int, V: int):
    """Achieved HBM bandwidth of the memory-bound kernels of the step, each timed alone with HIP
    events on the launch stream at the 7B shapes, against the 8 TB/s peak.  Bytes are algorithmic
    (every operand and result moved once).  Each kernel cycles over enough distinct buffers that
    nothing it reads is left in the 256 MB Infinity Cache from its previous launch."""
    import torch

    from olmax_amd import ops
    BF = torch.bfloat16
    dev = "cuda"
    out = []

    def timed(name, nbytes, footprint, make, call, iters=24):
        nset = max(2, int(768e6 // footprint) + 1)
        sets = [make() for _ in range(nset)]
        for i in range(4):
            call(sets[i % nset])
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(iters):
            call(sets[i % nset])
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / iters
        out.append({"kernel": name, "algorithmic_bytes": nbytes, "us": us, "achieved_GBps": nbytes / us / 1e3,
                    "frac_of_8TBps": nbytes / us / 1e3 / 8000.0})
        del sets
        torch.cuda.empty_cache()

    rnd = lambda *sh: torch.randn(*sh, device=dev).to(BF)
    w = torch.ones(d, device=dev, dtype=BF)
    # yardstick: what a plain device-to-device copy of the same size reaches under the same conditions
    timed("copy [T,d] bf16 (torch copy_, for scale)", 4 * T * d, 4 * T * d, lambda: (rnd(T, d), torch.empty(T, d, device=dev, dtype=BF)),
          lambda b: b[1].copy_(b[0]))
    timed("copy [T,F] x 5 arrays of bf16 (torch copy_, for scale)", 4 * T * F * 5 // 2, 4 * T * F * 5 // 2,
          lambda: (rnd(T, 5 * F // 2), torch.empty(T, 5 * F // 2, device=dev, dtype=BF)), lambda b: b[1].copy_(b[0]))
    timed("rmsnorm_fwd [T,d]", 4 * T * d, 4 * T * d, lambda: (rnd(T, d), torch.empty(T, d, device=dev, dtype=BF)),
          lambda b: ops.rms_norm_fwd(b[0], w, 1e-6, out=b[1]))
    dw = torch.zeros(d, device=dev)
    timed("rmsnorm_bwd + residual grad [T,d]", 8 * T * d, 8 * T * d,
          lambda: (rnd(T, d), rnd(T, d), rnd(T, d), torch.empty(T, d, device=dev, dtype=BF)),
          lambda b: ops.rms_norm_bwd(b[0], w, b[1], 1e-6, dres=b[2], dw=dw, out=b[3]))
    timed("glu_bwd (silu) [T,F]", 10 * T * F, 10 * T * F,
          lambda: (rnd(T, 2 * F), rnd(T, F), torch.empty(T, 2 * F, device=dev, dtype=BF)),
          lambda b: ops.glu_bwd(b[0][:, :F], b[0][:, F:], b[1], "silu", dgate=b[2][:, :F], dup=b[2][:, F:]))
    cos, sin = ops.rope_tables(4096, 128, 5e5, dev)
    timed("qk_rope_bwd in place [T,heads*128]", 4 * T * heads * 128, 2 * T * heads * 128, lambda: (rnd(T, heads * 128),),
          lambda b: ops.qk_rope_bwd(b[0], cos, sin, heads=heads, head_dim=128, seq_len=4096, out=b[0]))
    labels = torch.randint(0, V, (T,), device=dev, dtype=torch.int32)
    timed("cross_entropy fwd+bwd in place [T,V] bf16", 4 * T * V, 2 * T * V, lambda: (rnd(T, V),),
          lambda b: ops.cross_entropy(b[0], labels, inplace=True), iters=8)
    n = 202_383_360  # parameters of one 7B block
    timed("adamw (bf16 grads, bf16 copy out) one block", 28 * n, 30 * n,
          lambda: (torch.zeros(n, device=dev), rnd(n), torch.zeros(n, device=dev), torch.zeros(n, device=dev),
                   torch.empty(n, device=dev, dtype=BF)),
          lambda b: ops.adamw_(b[0], b[1], b[2], b[3], step=1, lr=1e-4, shadow=b[4]), iters=8)
    return out


def secondary_config(args):
    """The other BASELINE workloads at their real widths, as a clearly labelled secondary leg
    (--config 2 | 4 | 5; never the headline): ms per step and the share of the 2.5 PFLOP/s bf16
    peak the step's model FLOPs reach, beside the ideal step time.
      2: one OLMo2-7B block, forward + backward in isolation, activations [2, 4096, 4096];
      4: Gemma2-27B-like 4-layer slice + embedding + LM head + CE, forward + backward;
      5: Gemma3-27B-like 6-layer slice, forward + backward + the fused AdamW step."""
    import torch
    from olmax_amd import TransformerRecipe
    from olmax_amd.layer import TransformerBlock

    B, S = 2, 4096
    T = B * S
    gen = torch.Generator().manual_seed(0)
    k = args.config
    if k == 2:
        cfg = TransformerRecipe.olmo2_7B_block_bench()
        blk = TransformerBlock(cfg, batch_size=B, sequence_length=S)
        g = torch.Generator(device="cuda").manual_seed(0)
        for w in (blk.wqkv, blk.wo, blk.wgu, blk.wdown):
            w.normal_(0.0, 0.02, generator=g)
        x = torch.randn(T, cfg.d_model, device="cuda", generator=g).to(torch.bfloat16)
        dy = torch.randn(T, cfg.d_model, device="cuda", generator=g).to(torch.bfloat16)

        def step():
            blk.forward(x)
            blk.backward(dy)
        d, H, K, D, F = cfg.d_model, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim, cfg.hidden_size
        flops = 3.0 * T * (2 * d * (H + 2 * K) * D + 2 * H * D * d + 6 * d * F + 4 * H * D * (S + 1) / 2)
        what = ("one OLMo2-7B block forward+backward (configs[1]): d_model 4096, 32x128 heads, SwiGLU 11008, post-norm + "
                "head-wise QK-norm, theta 5e5, activations [2, 4096, 4096] bf16")
        params = blk.wqkv.numel() + blk.wo.numel() + blk.wgu.numel() + blk.wdown.numel()
    else:
        cfg = TransformerRecipe.gemma2_slice_bench() if k == 4 else TransformerRecipe.gemma3_slice_bench()
        model = cfg.build(batch_size=B, sequence_length=S, seed=0)
        ids = torch.randint(0, cfg.vocab_size, (T,), generator=gen, dtype=torch.int32).cuda()
        labels = torch.randint(0, cfg.vocab_size, (T,), generator=gen, dtype=torch.int32).cuda()
        count = [0]
        if k == 4:
            def step():
                model.loss_and_grads(ids, labels)
            what = ("Gemma2-27B-like 4-layer slice forward+backward (configs[3]): d_model 4608, 32/16 heads x 128, GeGLU 36864, "
                    "pre+post norm, 4096-window / global layers alternating, soft-caps 50 / 30, vocab 256000 tied, seq 4096, mb 2")
        else:
            def step():
                count[0] += 1
                model.train_step(ids, labels, step=count[0], lr=1e-4, b1=0.9, b2=0.95, weight_decay=0.1,
                                 no_decay_modules=["embedding.weight"], overlap_optimizer=not args.no_overlap)
            what = ("Gemma3-27B-like 6-layer slice forward+backward+AdamW (configs[4]): d_model 5376, 32/16 heads x 128, QK-norm, "
                    "1024-token windows on 5 of 6 layers, theta 1e4 / 1e6, GeGLU 21504, vocab 262144 tied, seq 4096, mb 2")
        flops = cfg.flops_per_token(S) * T
        params = model.num_params
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / max(1, args.steps) * 1e3
    ideal = flops / PEAK_BF16 * 1e3
    print(json.dumps({
        "metric": f"SECONDARY LEG (not the headline): ms/step and share of the bf16 peak, BASELINE configs[{k - 1}]",
        "value": T / ms * 1e3, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic (uniform tokens / N(0,1) activations, N(0,0.02) init, resident in HBM)",
        "mfu_bf16": ideal / ms, "tflop_per_step": flops / 1e12, "ideal_ms_at_2.5_PFLOPs": ideal,
        "config": {"workload": what, "params": params, "global_batch": B, "seq_len": S}}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--no-checkpoint", action="store_true", help="keep activations instead of full-block recompute")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-hbm-kernels", action="store_true", help="skip the stand-alone timing of the memory-bound kernels")
    ap.add_argument("--no-keep-activations-leg", action="store_true", help="skip the extra measurement without recompute")
    ap.add_argument("--no-overlap", action="store_true", help="run AdamW after the backward pass instead of overlapping it on a second stream")
    ap.add_argument("--profiler-ranges", action="store_true", help="emit roctx ranges per layer and phase (for rocprofv3 --marker-trace)")
    ap.add_argument("--config", type=int, default=3, choices=[2, 3, 4, 5],
                    help="BASELINE workload (1-based): 3 = the headline Llama-like 7B step (default); 2, 4, 5 = secondary legs")
    ap.add_argument("--layers", type=int, default=32, help="debug only: fewer layers (result is then not the headline metric)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures ONE MI355X only (no collectives or sharding); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from olmax_amd import AdamWConfig, Trainer, TransformerRecipe, WarmupCosineDecaySchedule, _lib

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(1)
    L = _lib.load()
    if args.config != 3:
        secondary_config(args)
        return
    if args.profiler_ranges:
        Trainer.set_profiler_ranges(True)
    B, S = 2, 4096
    cfg = TransformerRecipe.llama_like_7B_bench()
    cfg.num_layers = args.layers
    if args.no_checkpoint:
        cfg.layer_ac_policy = None
    model = cfg.build(batch_size=B, sequence_length=S, seed=0)
    # the reference benchmark's optimizer: AdamW, cosine 1e-6 -> 1e-4 -> 1e-6, embedding not decayed
    optim = AdamWConfig(lr=WarmupCosineDecaySchedule(warmup_steps=20, decay_steps=80, peak_value=1e-4,
                                                     init_value=1e-6, end_value=1e-6),
                        no_decay_modules=["embedding.weight"])
    trainer = Trainer(model, optim, overlap_optimizer=not args.no_overlap)
    T = B * S
    nb = 4
    gen = torch.Generator().manual_seed(0)
    batches = []
    for _ in range(nb):
        ids = torch.randint(0, cfg.vocab_size, (T,), generator=gen, dtype=torch.int32).cuda()
        labels = torch.randint(0, cfg.vocab_size, (T,), generator=gen, dtype=torch.int32).cuda()
        batches.append((ids, labels))

    losses = []
    for i in range(args.warmup):
        losses.append(trainer.process_microbatch(*batches[i % nb]))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        losses.append(trainer.process_microbatch(*batches[(args.warmup + i) % nb]))
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / max(1, args.steps) * 1e3
    tps = T * args.steps / dt
    flops_tok = cfg.flops_per_token(S)
    mfu = tps * flops_tok / PEAK_BF16
    losses = [float(l) if not hasattr(l, "item") else l.item() for l in losses[-1:]]

    # ---- roofline of the dominant kernel: one more (untimed) step with a HIP-event pair around
    # every GEMM launch, recorded on the launch stream
    L.olmax_gemm_profile_begin()
    trainer.process_microbatch(*batches[0])
    torch.cuda.synchronize()
    cap = 64
    keys = (ctypes.c_int32 * cap)(); ms = (ctypes.c_double * cap)(); fl = (ctypes.c_double * cap)()
    by = (ctypes.c_double * cap)(); ln = (ctypes.c_int64 * cap)()
    n = L.olmax_gemm_profile_end(keys, ms, fl, by, ln, cap)
    per = []
    for i in range(n):
        k = keys[i]
        name = "gemm_bf16_kernel<tile%d,%s,%s%s%s%s>" % (k & 0xfff, "A_KC" if k >> 12 & 1 else "A_MC", "B_KC" if k >> 13 & 1 else "B_NC",
                                                         ",res" if k >> 14 & 1 else "", ",f32out" if k >> 15 & 1 else "",
                                                         ",glu" if k >> 16 & 1 else ",rope" if k >> 17 & 1 else "")
        per.append({"kernel": name, "key": k, "launches": ln[i], "total_ms": ms[i], "avg_ms": ms[i] / ln[i],
                    "tflops": fl[i] / ms[i] / 1e9, "algorithmic_bytes_per_launch": by[i] / ln[i]})
    per.sort(key=lambda r: -r["total_ms"])
    dom = per[0] if per else None
    gemm_ms = sum(r["total_ms"] for r in per)
    gemm_fl = sum(r["tflops"] * r["total_ms"] for r in per)  # TFLOP*1e-3... (tflops * ms = GFLOP)
    roofline = None
    if dom:
        roofline = {"bound": "mfma", "achieved": dom["tflops"], "peak": PEAK_BF16 / 1e12, "unit": "TFLOP/s",
                    "frac": dom["tflops"] / (PEAK_BF16 / 1e12),
                    "traffic": gemm_traffic_bytes().get(dom["key"]),
                    "traffic_source": f"{TRAFFIC_PROFILE} (two rocprofv3 --pmc runs of this script, FETCH_SIZE then WRITE_SIZE, "
                                      "scaled by what a cast kernel of known size reads in the same runs; not re-measured by this run)",
                    "algorithmic_bytes": dom["algorithmic_bytes_per_launch"], "kernel": dom["kernel"],
                    "avg_launch_ms": dom["avg_ms"], "launches_per_step": dom["launches"],
                    "all_gemm": {"ms_per_step": gemm_ms, "tflops": gemm_fl / gemm_ms if gemm_ms else None,
                                 "share_of_step": gemm_ms / ms_per_step}}

    out = {
        "metric": "train tokens/sec + bf16 MFU, Llama-like 7B seq 4096 mb=2, 1 MI355X",
        "value": tps, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic (uniform tokens, N(0,0.02) init, resident in HBM)",
        "mfu_bf16": mfu, "gflop_per_token": flops_tok / 1e9, "last_loss": losses[-1],
        "config": {"workload": "Llama-like 7B full train step (configs[2]): 32 layers, d_model 4096, 32x128 heads, "
                               "SwiGLU 11008, vocab 100352 untied, seq 4096, micro-batch 2, bf16 compute, fp32 master + "
                               "AdamW, " + ("activations kept (no recompute)" if args.no_checkpoint else "full-block activation checkpointing"),
                   "layers": cfg.num_layers, "global_batch": B, "seq_len": S, "params": model.num_params,
                   "activation_checkpointing": not args.no_checkpoint, "optimizer_overlap": not args.no_overlap},
        "roofline": roofline,
        "gemm_kernels": per[:6],
    }
    if not args.no_checkpoint and not args.no_keep_activations_leg:
        # Same model, same step, but every block keeps its activations (34.8 GB of the 288 GB)
        # instead of recomputing them: reported beside the headline value, never as it.
        model.c.checkpoint = 0
        model._workspace = None
        torch.cuda.empty_cache()
        for i in range(max(1, args.warmup)):
            trainer.process_microbatch(*batches[i % nb])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            trainer.process_microbatch(*batches[i % nb])
        torch.cuda.synchronize()
        dt2 = time.perf_counter() - t0
        tps2 = T * args.steps / dt2
        out["keep_activations"] = {"value": tps2, "unit": "tokens/s", "ms_per_step": dt2 / args.steps * 1e3,
                                   "mfu_bf16": tps2 * flops_tok / PEAK_BF16,
                                   "note": "activation_checkpointing off (reference recipe default); not the headline config"}
    if not args.no_hbm_kernels:
        del trainer, model
        torch.cuda.empty_cache()
        out["hbm_kernels"] = hbm_kernels(T, cfg.d_model, 11008, 64, cfg.vocab_size)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
