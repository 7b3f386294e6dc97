"""Host-side mirror of the reference's model API for the HIP hot path.

``TransformerConfig`` / ``Transformer`` / ``TransformerRecipe`` follow the reference's names
and argument meaning (src/olmax/nn/transformer/model.py:24-213, recipes.py:38-360, the layer
classes of layer.py:20-185 and MultiheadSelfAttentionConfig of attention.py:325-376) with the
nested layer/attention configs flattened into one dataclass.  All parameters live in ONE flat
fp32 master buffer plus a flat bf16 working copy on the GPU (laid out by the C library so
that q/k/v and gate/up are adjacent and fuse into single GEMMs); ``named_parameters()``
exposes per-leaf views under the reference's pytree paths.  Every computation is done by
libolmax_hip through its C ABI; this file only owns device memory.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import torch

from . import _lib, ops
from ._lib import check, f32, i32, i64, ptr, stream_ptr

LAYER_TYPES = {"default": 0, "reordered_norm": 1, "gemma": 2}
ACTIVATIONS = {"silu": 0, "gelu": 1}


class CModelConfig(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in (
        "vocab", "d_model", "n_layers", "n_heads", "n_kv_heads", "head_dim", "hidden", "layer_type", "act",
        "qk_norm", "tied", "batch", "seq_len", "checkpoint")] + [(n, ctypes.c_float) for n in (
        "eps", "attn_softcap", "final_softcap")]


class CLeaf(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("layer", ctypes.c_int32), ("offset", ctypes.c_int64),
                ("numel", ctypes.c_int64), ("rows", ctypes.c_int32), ("cols", ctypes.c_int32),
                ("grad_f32", ctypes.c_int32), ("grad_f32_offset", ctypes.c_int64)]


class CBlockWeights(ctypes.Structure):
    _fields_ = [(n, ctypes.c_void_p) for n in ("wqkv", "wo", "wgu", "wdown", "attn_norm", "mlp_norm",
                                                "attn_in_norm", "mlp_in_norm", "q_norm", "k_norm")]


class CBlockGrads(ctypes.Structure):
    _fields_ = [(n, ctypes.c_void_p) for n in ("wqkv", "wo", "wgu", "wdown", "attn_norm", "mlp_norm",
                                                "attn_in_norm", "mlp_in_norm", "q_norm", "k_norm")]


_LEAF_NAMES = {
    0: "embedding.weight", 1: "layers.{l}.attention.q_proj.weight", 2: "layers.{l}.attention.k_proj.weight",
    3: "layers.{l}.attention.v_proj.weight", 4: "layers.{l}.attention.o_proj.weight",
    5: "layers.{l}.mlp.gate_proj.weight", 6: "layers.{l}.mlp.up_proj.weight", 7: "layers.{l}.mlp.down_proj.weight",
    8: "layers.{l}.attention_norm.weight", 9: "layers.{l}.mlp_norm.weight",
    10: "layers.{l}.attention_input_norm.weight", 11: "layers.{l}.mlp_input_norm.weight",
    12: "layers.{l}.attention.q_norm.weight", 13: "layers.{l}.attention.k_norm.weight",
    14: "norm.weight", 15: "lm_head.proj.weight",
}
_NORM_KINDS = {8, 9, 10, 11, 12, 13, 14}


@dataclass
class TransformerConfig:
    vocab_size: int
    d_model: int
    hidden_size: int
    num_layers: int
    n_heads: int
    n_kv_heads: Optional[int] = None
    head_dim: Optional[int] = None
    layer_type: str = "default"            # "default" | "reordered_norm" | "gemma"
    activation: str = "silu"               # "silu" | "gelu" (tanh approximation)
    qk_norm_headwise: bool = False         # QK-norm with one weight [head_dim] shared by the heads (attention.py:293-296)
    qk_norm: Optional[bool] = None         # None: on iff qk_norm_headwise; True with qk_norm_headwise False:
                                           # full-width QK-norm before the reshape (attention.py:281-284)
    norm_eps: float = 1e-5                 # RMSNormConfig default, normalization.py:95
    rope_theta: float = 10_000.0
    rope_theta_per_layer: Optional[Sequence[float]] = None
    window_size: Optional[int] = None      # one static window for every layer, as the reference
    window_size_per_layer: Optional[Sequence[Optional[int]]] = None
    attn_logit_softcap: float = 0.0
    final_logit_softcap: float = 0.0
    tie_embeddings: bool = False
    layer_ac_policy: Optional[str] = None  # "nothing_saveable" = full-block recompute

    def __post_init__(self):
        if self.n_kv_heads is None:
            self.n_kv_heads = self.n_heads
        if self.head_dim is None:
            self.head_dim = self.d_model // self.n_heads
        if self.layer_type not in LAYER_TYPES:
            raise ValueError(f"unknown layer_type {self.layer_type!r}")
        if self.activation not in ACTIVATIONS:
            raise ValueError(f"unknown activation {self.activation!r}")
        if self.qk_norm is None:
            self.qk_norm = self.qk_norm_headwise
        if self.qk_norm_headwise and not self.qk_norm:
            raise ValueError("qk_norm_headwise needs qk_norm")
        if self.layer_ac_policy not in (None, "nothing_saveable"):
            raise ValueError("layer_ac_policy must be None or 'nothing_saveable' (full block)")

    def windows(self) -> List[int]:
        if self.window_size_per_layer is not None:
            assert len(self.window_size_per_layer) == self.num_layers
            return [-1 if w is None else int(w) for w in self.window_size_per_layer]
        return [-1 if self.window_size is None else int(self.window_size)] * self.num_layers

    def qk_norm_mode(self) -> int:
        """0 off, 1 head-wise, 2 full width (olmax_model_config.qk_norm)."""
        return 0 if not self.qk_norm else (1 if self.qk_norm_headwise else 2)

    def thetas(self) -> List[float]:
        if self.rope_theta_per_layer is not None:
            assert len(self.rope_theta_per_layer) == self.num_layers
            return [float(t) for t in self.rope_theta_per_layer]
        return [float(self.rope_theta)] * self.num_layers

    def c_config(self, batch: int, seq_len: int) -> CModelConfig:
        return CModelConfig(
            vocab=self.vocab_size, d_model=self.d_model, n_layers=self.num_layers, n_heads=self.n_heads,
            n_kv_heads=self.n_kv_heads, head_dim=self.head_dim, hidden=self.hidden_size,
            layer_type=LAYER_TYPES[self.layer_type], act=ACTIVATIONS[self.activation],
            qk_norm=self.qk_norm_mode(), tied=int(self.tie_embeddings), batch=batch, seq_len=seq_len,
            checkpoint=int(self.layer_ac_policy == "nothing_saveable"), eps=self.norm_eps,
            attn_softcap=self.attn_logit_softcap, final_softcap=self.final_logit_softcap)

    def build(self, *, batch_size: int, sequence_length: int, seed: int = 0, device="cuda") -> "Transformer":
        return Transformer(self, batch_size=batch_size, sequence_length=sequence_length, seed=seed, device=device)

    def flops_per_token(self, seq_len: int) -> float:
        """Model FLOPs of one training token: 3 x forward; matmul 2MNK; attention counted at
        its exact number of visible (query, key) pairs."""
        d, H, K, D, F, V = self.d_model, self.n_heads, self.n_kv_heads, self.head_dim, self.hidden_size, self.vocab_size
        per_layer = 2 * d * (H * D + 2 * K * D) + 2 * H * D * d + 3 * 2 * d * F
        attn = 0.0
        for w in self.windows():
            pairs = sum(min(i, w) + 1 for i in range(seq_len)) if w >= 0 else seq_len * (seq_len + 1) / 2
            attn += 4 * H * D * pairs / seq_len
        fwd = self.num_layers * per_layer + attn + 2 * d * V
        return 3.0 * fwd


class TransformerRecipe:
    """Named model configurations (src/olmax/nn/transformer/recipes.py) plus the two
    benchmark variants this repository is measured on."""

    @staticmethod
    def llama_like_7B(vocab_size: int = 50_304, rope_theta: float = 10_000.0) -> TransformerConfig:
        return TransformerConfig(vocab_size=vocab_size, d_model=4096, hidden_size=11008, num_layers=32, n_heads=32,
                                 rope_theta=rope_theta)

    @staticmethod
    def llama_like_7B_bench() -> TransformerConfig:
        """The measured configuration: vocab 100352, theta 5e5, eps 1e-6, full-block AC."""
        c = TransformerRecipe.llama_like_7B(vocab_size=100_352, rope_theta=500_000.0)
        c.norm_eps = 1e-6
        c.layer_ac_policy = "nothing_saveable"
        return c

    @staticmethod
    def llama_like_271M() -> TransformerConfig:
        return TransformerConfig(vocab_size=50_304, d_model=1024, hidden_size=2816, num_layers=16, n_heads=8)

    @staticmethod
    def llama3_8B() -> TransformerConfig:
        """recipes.py:126-165 (GQA 32/8 heads, theta 5e5, vocab 128256, hidden 14336)."""
        return TransformerConfig(vocab_size=128_256, d_model=4096, hidden_size=14_336, num_layers=32, n_heads=32,
                                 n_kv_heads=8, rope_theta=500_000.0)

    @staticmethod
    def llama3_70B() -> TransformerConfig:
        """recipes.py:168-200 (d 8192, 80 layers, GQA 64/8, full-block AC).  Its fp32 master
        parameters and Adam moments (70.6 B x 12 B) do not fit one 288 GB GPU: sizes only."""
        return TransformerConfig(vocab_size=128_256, d_model=8192, hidden_size=28_672, num_layers=80, n_heads=64,
                                 n_kv_heads=8, rope_theta=500_000.0, layer_ac_policy="nothing_saveable")

    @staticmethod
    def olmo2_32B() -> TransformerConfig:
        """recipes.py:246-282 (reordered norm, head-wise QK-norm, GQA 40/8, full-block AC)."""
        return TransformerConfig(vocab_size=100_278, d_model=5120, hidden_size=27_648, num_layers=64, n_heads=40,
                                 n_kv_heads=8, layer_type="reordered_norm", qk_norm_headwise=True,
                                 layer_ac_policy="nothing_saveable")

    @staticmethod
    def olmo2_7B() -> TransformerConfig:
        return TransformerConfig(vocab_size=100_278, d_model=4096, hidden_size=11008, num_layers=32, n_heads=32,
                                 layer_type="reordered_norm", qk_norm_headwise=True)

    @staticmethod
    def gemma2_like_27B(num_layers: int = 46) -> TransformerConfig:
        return TransformerConfig(vocab_size=256_000, d_model=4608, hidden_size=36864, num_layers=num_layers,
                                 n_heads=32, n_kv_heads=16, head_dim=128, layer_type="gemma", activation="gelu")

    @staticmethod
    def gemma3_like_27B(num_layers: int = 62) -> TransformerConfig:
        return TransformerConfig(vocab_size=256_000, d_model=5376, hidden_size=21504, num_layers=num_layers,
                                 n_heads=32, n_kv_heads=16, head_dim=128, layer_type="gemma", activation="gelu",
                                 qk_norm_headwise=True)

    # ---- the other measured / parity-tested workloads, at their real widths
    @staticmethod
    def olmo2_7B_block_bench() -> TransformerConfig:
        """One OLMo2-7B block in isolation (ReorderedNormTransformerLayer, layer.py:102-116, with
        head-wise QK-norm): d 4096, 32 x 128 heads, SwiGLU 11008, eps 1e-6, theta 5e5."""
        c = TransformerRecipe.olmo2_7B()
        c.num_layers, c.norm_eps, c.rope_theta, c.vocab_size = 1, 1e-6, 500_000.0, 8
        return c

    @staticmethod
    def gemma2_slice_bench(num_layers: int = 4) -> TransformerConfig:
        """Gemma2-27B-like slice: d 4608, 32 / 16 heads x 128, GeGLU 36864, pre+post norm, layers
        alternating a 4096-token window and global attention, attention soft-cap 50, final soft-cap
        30, vocab 256000 tied, full-block recompute."""
        c = TransformerRecipe.gemma2_like_27B(num_layers)
        c.norm_eps, c.rope_theta = 1e-6, 10_000.0
        c.window_size_per_layer = [4096 if l % 2 == 0 else None for l in range(num_layers)]
        c.attn_logit_softcap, c.final_logit_softcap, c.tie_embeddings = 50.0, 30.0, True
        c.layer_ac_policy = "nothing_saveable"
        return c

    @staticmethod
    def gemma3_slice_bench(num_layers: int = 6) -> TransformerConfig:
        """Gemma3-27B-like slice (5 local : 1 global): d 5376, 32 / 16 heads x 128, head-wise QK-norm,
        1024-token windows and theta 1e4 on local layers, theta 1e6 on the global one, GeGLU 21504,
        vocab 262144 tied, full-block recompute."""
        c = TransformerRecipe.gemma3_like_27B(num_layers)
        c.vocab_size, c.norm_eps = 262_144, 1e-6
        glob = [(l + 1) % 6 == 0 for l in range(num_layers)]
        c.window_size_per_layer = [None if g else 1024 for g in glob]
        c.rope_theta_per_layer = [1e6 if g else 1e4 for g in glob]
        c.tie_embeddings = True
        c.layer_ac_policy = "nothing_saveable"
        return c

    @staticmethod
    def tiny_llama() -> TransformerConfig:
        """4 layers, d 256, 4x64 heads, hidden 1024, vocab 4096 (CPU-sized plumbing config)."""
        return TransformerConfig(vocab_size=4096, d_model=256, hidden_size=1024, num_layers=4, n_heads=4,
                                 norm_eps=1e-6, rope_theta=10_000.0)


class Transformer:
    """Flat-buffer model on one GPU.  ``loss_and_grads`` = compute_loss_and_grads,
    ``adamw_step`` = step_optimizer (src/olmax/train/trainer.py:723-757)."""

    def __init__(self, config: TransformerConfig, *, batch_size: int, sequence_length: int, seed: int = 0,
                 device="cuda", init_std: float = 0.02):
        if not torch.cuda.is_available():
            raise _lib.OlmaxHipError("olmax_amd.Transformer needs a GPU: the HIP path has no CPU fallback")
        self.config = config
        self.batch_size, self.sequence_length = batch_size, sequence_length
        self.device = torch.device(device)
        self._L = _lib.load()
        L = self._L
        for fn in ("olmax_model_num_params", "olmax_model_grad_f32_elems", "olmax_model_workspace_bytes",
                   "olmax_block_acts_bytes", "olmax_block_tmp_bytes"):
            getattr(L, fn).restype = ctypes.c_int64
        self.c = config.c_config(batch_size, sequence_length)
        self.num_params = L.olmax_model_num_params(ctypes.byref(self.c))
        if self.num_params < 0:
            raise _lib.OlmaxHipError(L.olmax_last_error_string().decode())
        n_leaf = L.olmax_model_layout(ctypes.byref(self.c), None, 0)
        arr = (CLeaf * n_leaf)()
        L.olmax_model_layout(ctypes.byref(self.c), arr, n_leaf)
        self.leaves = list(arr)
        self.grad_f32_elems = L.olmax_model_grad_f32_elems(ctypes.byref(self.c))

        dev = self.device
        self.master = torch.empty(self.num_params, device=dev, dtype=torch.float32)
        self.params_bf16 = torch.empty(self.num_params, device=dev, dtype=torch.bfloat16)
        self.grad_bf16 = torch.zeros(self.num_params, device=dev, dtype=torch.bfloat16)
        self.grad_f32 = torch.zeros(self.grad_f32_elems, device=dev, dtype=torch.float32)
        self.m: Optional[torch.Tensor] = None
        self.v: Optional[torch.Tensor] = None
        self.loss = torch.zeros((), device=dev, dtype=torch.float32)
        self.norm_scratch = torch.zeros(2, device=dev, dtype=torch.float32)
        self.grad_acc = None  # fp32 running mean over micro-batches, allocated on first use
        self._workspace: Optional[torch.Tensor] = None
        self._opt_stream = None
        self._decay_masks: Dict[tuple, object] = {}

        # per-layer windows and RoPE tables (get_buffer_cache, model.py:138-144)
        self._windows = (ctypes.c_int32 * max(1, config.num_layers))(*config.windows())
        tables: Dict[float, tuple] = {}
        for th in config.thetas():
            if th not in tables:
                tables[th] = ops.rope_tables(sequence_length, config.head_dim, th, dev)
        self.buffer_cache = tables
        self._cos = (ctypes.c_void_p * max(1, config.num_layers))(*[tables[t][0].data_ptr() for t in config.thetas()])
        self._sin = (ctypes.c_void_p * max(1, config.num_layers))(*[tables[t][1].data_ptr() for t in config.thetas()])
        self.reset_parameters(seed, init_std)

    # ------------------------------------------------------------------ parameters
    def leaf_name(self, leaf: CLeaf) -> str:
        return _LEAF_NAMES[leaf.kind].format(l=leaf.layer)

    def reset_parameters(self, seed: int = 0, std: float = 0.02) -> None:
        """N(0, std) for matrices, ones for norm weights (device RNG; reproducible per seed)."""
        g = torch.Generator(device=self.device).manual_seed(seed)
        for leaf in self.leaves:
            view = self.master[leaf.offset: leaf.offset + leaf.numel]
            if leaf.kind in _NORM_KINDS:
                view.fill_(1.0)
            else:
                view.normal_(0.0, std, generator=g)
        self.sync_working_copy()

    def sync_working_copy(self) -> None:
        """bf16 working copy <- fp32 master (cast_tree(params, bf16), trainer.py:728); afterwards
        the fused AdamW keeps it current."""
        check(self._L.olmax_cast_f32_to_bf16(stream_ptr(), ptr(self.master), ptr(self.params_bf16), i64(self.num_params)))

    def weight_decay_mask(self, no_decay_modules: Optional[Sequence[str]]):
        """OptimConfig.build_weight_decay_mask (src/olmax/optim/config.py:94-122) over this model's
        leaves: a ctypes int32 array in layout order, 0 where the dotted leaf path matches one of the
        fnmatch patterns (None when nothing is masked).  A pattern that matches nothing warns."""
        import fnmatch
        import warnings

        pats = tuple(no_decay_modules or ())
        if not pats:
            return None
        if pats not in self._decay_masks:
            names = [self.leaf_name(l) for l in self.leaves]
            for pat in pats:
                if not any(fnmatch.fnmatch(n, pat) for n in names):
                    warnings.warn(f"no decay pattern '{pat}' did not match any parameters")
            mask = [0 if any(fnmatch.fnmatch(n, pat) for pat in pats) else 1 for n in names]
            self._decay_masks[pats] = (ctypes.c_int32 * len(mask))(*mask)
        return self._decay_masks[pats]

    def named_parameters(self) -> Dict[str, torch.Tensor]:
        return {self.leaf_name(l): self.master[l.offset: l.offset + l.numel].view(l.rows, l.cols) if l.rows > 1
                else self.master[l.offset: l.offset + l.numel] for l in self.leaves}

    def named_gradients(self) -> Dict[str, torch.Tensor]:
        """Gradients of the last ``loss_and_grads`` call as fp32 tensors (cast_tree(grads, fp32))."""
        out = {}
        for l in self.leaves:
            if l.grad_f32:
                g = self.grad_f32[l.grad_f32_offset: l.grad_f32_offset + l.numel]
            else:
                g = self.grad_bf16[l.offset: l.offset + l.numel].float()
            out[self.leaf_name(l)] = g.view(l.rows, l.cols) if l.rows > 1 else g
        return out

    def load_state_dict(self, state: Dict[str, torch.Tensor]) -> None:
        names = {self.leaf_name(l): l for l in self.leaves}
        missing = set(names) - set(state)
        if missing:
            raise KeyError(f"missing parameters: {sorted(missing)[:5]}")
        for name, l in names.items():
            t = state[name].to(device=self.device, dtype=torch.float32).reshape(-1)
            if t.numel() != l.numel:
                raise ValueError(f"{name}: expected {l.numel} elements, got {t.numel()}")
            self.master[l.offset: l.offset + l.numel].copy_(t)
        self.sync_working_copy()

    # ------------------------------------------------------------------ compute
    def workspace(self) -> torch.Tensor:
        if self._workspace is None:
            n = self._L.olmax_model_workspace_bytes(ctypes.byref(self.c))
            self._workspace = torch.empty(n, device=self.device, dtype=torch.uint8)
        return self._workspace

    def _check_batch(self, ids, labels):
        T = self.batch_size * self.sequence_length
        for t in (ids, labels):
            if t.dtype != torch.int32 or t.numel() != T or not t.is_cuda or not t.is_contiguous():
                raise ValueError(f"ids/labels must be contiguous int32 GPU tensors of {T} elements")

    def loss_and_grads(self, ids: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
        """One micro-batch: forward, CE loss, full backward.  Returns the device loss scalar."""
        self._check_batch(ids, labels)
        ws = self.workspace()
        check(self._L.olmax_model_loss_and_grads(
            stream_ptr(), ctypes.byref(self.c), self._windows, self._cos, self._sin, ptr(self.params_bf16),
            ptr(ids), ptr(labels), ptr(self.loss), ptr(self.grad_bf16), ptr(self.grad_f32), ptr(ws), i64(ws.numel())))
        return self.loss

    def forward_loss(self, ids: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
        self._check_batch(ids, labels)
        ws = self.workspace()
        check(self._L.olmax_model_loss(
            stream_ptr(), ctypes.byref(self.c), self._windows, self._cos, self._sin, ptr(self.params_bf16),
            ptr(ids), ptr(labels), ptr(self.loss), ptr(ws), i64(ws.numel())))
        return self.loss

    def train_step(self, ids: torch.Tensor, labels: torch.Tensor, *, step: int, lr: float, b1: float = 0.9,
                   b2: float = 0.999, eps: float = 1e-8, weight_decay: float = 1e-4,
                   no_decay_modules: Optional[Sequence[str]] = None, max_grad_norm: Optional[float] = None,
                   overlap_optimizer: bool = True, hyper_dev: Optional[torch.Tensor] = None) -> torch.Tensor:
        """loss + gradients + AdamW in one library call (process_microbatch).  With
        ``overlap_optimizer`` each layer's AdamW runs on a second (default-priority) stream while
        the backward pass continues."""
        self._check_batch(ids, labels)
        if self.m is None:
            self.init_optimizer_state()
        ws = self.workspace()
        opt = None
        if overlap_optimizer and not max_grad_norm:
            if self._opt_stream is None:
                self._opt_stream = torch.cuda.Stream(device=self.device)
            opt = ctypes.c_void_p(self._opt_stream.cuda_stream)
        check(self._L.olmax_model_train_step(
            stream_ptr(), opt, ctypes.byref(self.c), self._windows, self._cos, self._sin, ptr(self.master), ptr(self.m),
            ptr(self.v), ptr(self.params_bf16), ptr(ids), ptr(labels), ptr(self.loss), ptr(self.grad_bf16),
            ptr(self.grad_f32), ptr(ws), i64(ws.numel()), i64(step), f32(lr), f32(b1), f32(b2), f32(eps),
            f32(weight_decay), self.weight_decay_mask(no_decay_modules), f32(max_grad_norm or 0.0), ptr(self.norm_scratch), ptr(hyper_dev)))
        return self.loss

    def accumulate_grads(self, mini_step: int) -> None:
        """Fold the gradients of the micro-batch just differentiated into the running mean
        ``self.grad_acc`` (fp32, parameter layout): optax.MultiSteps' accumulator, reference
        src/olmax/optim/config.py:153-154.  ``mini_step`` is 0-based inside the batch."""
        if self.grad_acc is None:
            self.grad_acc = torch.zeros(self.num_params, device=self.device, dtype=torch.float32)
        check(self._L.olmax_model_grad_accumulate(stream_ptr(), ctypes.byref(self.c), ptr(self.grad_acc),
                                                  ptr(self.grad_bf16), ptr(self.grad_f32), i32(mini_step)))

    def adamw_step_accumulated(self, *, step: int, lr: float, b1: float = 0.9, b2: float = 0.999, eps: float = 1e-8,
                               weight_decay: float = 1e-4, no_decay_modules: Optional[Sequence[str]] = None,
                               max_grad_norm: Optional[float] = None, hyper_dev: Optional[torch.Tensor] = None) -> None:
        """AdamW (and the optional global-norm clip) on the accumulated mean gradient."""
        if self.m is None:
            self.init_optimizer_state()
        if self.grad_acc is None:
            raise ValueError("adamw_step_accumulated: no gradients have been accumulated")
        check(self._L.olmax_model_adamw_accumulated(
            stream_ptr(), ctypes.byref(self.c), ptr(self.master), ptr(self.m), ptr(self.v), ptr(self.params_bf16),
            ptr(self.grad_acc), i64(step), f32(lr), f32(b1), f32(b2), f32(eps), f32(weight_decay),
            self.weight_decay_mask(no_decay_modules), f32(max_grad_norm or 0.0), ptr(self.norm_scratch), ptr(hyper_dev)))

    def init_optimizer_state(self) -> None:
        self.m = torch.zeros(self.num_params, device=self.device, dtype=torch.float32)
        self.v = torch.zeros(self.num_params, device=self.device, dtype=torch.float32)

    def adamw_step(self, *, step: int, lr: float, b1: float = 0.9, b2: float = 0.999, eps: float = 1e-8,
                   weight_decay: float = 1e-4, no_decay_modules: Optional[Sequence[str]] = None,
                   max_grad_norm: Optional[float] = None, hyper_dev: Optional[torch.Tensor] = None):
        """``hyper_dev``: optional fp32 GPU tensor {lr, 1 - b1^step, 1 - b2^step} that replaces the host
        ``step`` / ``lr`` (schedules that live on the device)."""
        if self.m is None:
            self.init_optimizer_state()
        check(self._L.olmax_model_adamw(
            stream_ptr(), ctypes.byref(self.c), ptr(self.master), ptr(self.m), ptr(self.v), ptr(self.params_bf16),
            ptr(self.grad_bf16), ptr(self.grad_f32), i64(step), f32(lr), f32(b1), f32(b2), f32(eps), f32(weight_decay),
            self.weight_decay_mask(no_decay_modules), f32(max_grad_norm or 0.0), ptr(self.norm_scratch), ptr(hyper_dev)))
