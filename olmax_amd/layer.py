"""One transformer block in isolation on the HIP path (olmax_block_fwd / olmax_block_bwd).

Mirrors ``TransformerLayer`` / ``ReorderedNormTransformerLayer`` / ``GemmaTransformerLayer``
(src/olmax/nn/transformer/layer.py:20-185): ``forward(x)`` then ``backward(dy)`` returns the
input gradient and fills ``grads`` for every leaf, named as in the reference pytree.
"""
from __future__ import annotations

import ctypes
from typing import Dict, Optional

import torch

from . import _lib, ops
from ._lib import check, i32, i64, ptr, stream_ptr
from .transformer import CBlockGrads, CBlockWeights, TransformerConfig

BF16 = torch.bfloat16


class TransformerBlock:
    def __init__(self, config: TransformerConfig, *, batch_size: int, sequence_length: int, layer_idx: int = 0,
                 device="cuda"):
        if not torch.cuda.is_available():
            raise _lib.OlmaxHipError("olmax_amd.TransformerBlock needs a GPU: the HIP path has no CPU fallback")
        self.config, self.B, self.S = config, batch_size, sequence_length
        self.device = torch.device(device)
        self._L = _lib.load()
        self._L.olmax_block_acts_bytes.restype = ctypes.c_int64
        self._L.olmax_block_tmp_bytes.restype = ctypes.c_int64
        self.c = config.c_config(batch_size, sequence_length)
        c = config
        d, H, K, D, F = c.d_model, c.n_heads, c.n_kv_heads, c.head_dim, c.hidden_size
        dev = self.device
        self.wqkv = torch.zeros((H + 2 * K) * D, d, device=dev, dtype=BF16)
        self.wo = torch.zeros(d, H * D, device=dev, dtype=BF16)
        self.wgu = torch.zeros(2 * F, d, device=dev, dtype=BF16)
        self.wdown = torch.zeros(d, F, device=dev, dtype=BF16)
        self.norms: Dict[str, torch.Tensor] = {"attention_norm": torch.ones(d, device=dev, dtype=BF16),
                                               "mlp_norm": torch.ones(d, device=dev, dtype=BF16)}
        if c.layer_type == "gemma":
            self.norms["attention_input_norm"] = torch.ones(d, device=dev, dtype=BF16)
            self.norms["mlp_input_norm"] = torch.ones(d, device=dev, dtype=BF16)
        if c.qk_norm:  # head-wise: one weight [D]; full width: [H*D] for q, [K*D] for k
            self.norms["attention.q_norm"] = torch.ones(D if c.qk_norm_headwise else H * D, device=dev, dtype=BF16)
            self.norms["attention.k_norm"] = torch.ones(D if c.qk_norm_headwise else K * D, device=dev, dtype=BF16)
        self.window = c.windows()[layer_idx] if c.num_layers > layer_idx else (-1 if c.window_size is None else c.window_size)
        theta = c.thetas()[layer_idx] if c.num_layers > layer_idx else c.rope_theta
        self.cos, self.sin = ops.rope_tables(sequence_length, D, theta, dev)
        self.acts = torch.empty(self._L.olmax_block_acts_bytes(ctypes.byref(self.c)), device=dev, dtype=torch.uint8)
        self.tmp: Optional[torch.Tensor] = None
        self._x: Optional[torch.Tensor] = None
        self.grads: Dict[str, torch.Tensor] = {}

    def load_state_dict(self, state: Dict[str, torch.Tensor]) -> None:
        """Keys as in the reference: attention.{q,k,v,o}_proj.weight, mlp.{gate,up,down}_proj.weight, *_norm.weight."""
        c = self.config
        HD, KD, F = c.n_heads * c.head_dim, c.n_kv_heads * c.head_dim, c.hidden_size
        g = lambda k: state[k].to(device=self.device, dtype=BF16)
        self.wqkv[:HD].copy_(g("attention.q_proj.weight"))
        self.wqkv[HD:HD + KD].copy_(g("attention.k_proj.weight"))
        self.wqkv[HD + KD:].copy_(g("attention.v_proj.weight"))
        self.wo.copy_(g("attention.o_proj.weight"))
        self.wgu[:F].copy_(g("mlp.gate_proj.weight"))
        self.wgu[F:].copy_(g("mlp.up_proj.weight"))
        self.wdown.copy_(g("mlp.down_proj.weight"))
        for name in self.norms:
            self.norms[name].copy_(g(name + ".weight"))

    def _weights(self) -> CBlockWeights:
        n = self.norms
        p = lambda k: n[k].data_ptr() if k in n else None
        return CBlockWeights(wqkv=self.wqkv.data_ptr(), wo=self.wo.data_ptr(), wgu=self.wgu.data_ptr(),
                             wdown=self.wdown.data_ptr(), attn_norm=p("attention_norm"), mlp_norm=p("mlp_norm"),
                             attn_in_norm=p("attention_input_norm"), mlp_in_norm=p("mlp_input_norm"),
                             q_norm=p("attention.q_norm"), k_norm=p("attention.k_norm"))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        assert x.is_cuda and x.dtype == BF16 and x.is_contiguous() and x.numel() == self.B * self.S * self.config.d_model
        y = torch.empty_like(x)
        w = self._weights()
        check(self._L.olmax_block_fwd(stream_ptr(), ctypes.byref(self.c), ctypes.byref(w), i32(self.window),
                                      ptr(self.cos), ptr(self.sin), ptr(x), ptr(y), ptr(self.acts), i64(self.acts.numel())))
        self._x = x
        return y

    def backward(self, dy: torch.Tensor) -> torch.Tensor:
        assert self._x is not None, "call forward first"
        assert dy.is_cuda and dy.dtype == BF16 and dy.is_contiguous()
        if self.tmp is None:
            self.tmp = torch.empty(self._L.olmax_block_tmp_bytes(ctypes.byref(self.c)), device=self.device, dtype=torch.uint8)
        dev = self.device
        c = self.config
        HD, KD, F = c.n_heads * c.head_dim, c.n_kv_heads * c.head_dim, c.hidden_size
        gqkv, go, ggu, gdown = (torch.empty_like(t) for t in (self.wqkv, self.wo, self.wgu, self.wdown))
        gn = {k: torch.zeros(v.numel(), device=dev, dtype=torch.float32) for k, v in self.norms.items()}
        p = lambda k: gn[k].data_ptr() if k in gn else None
        g = CBlockGrads(wqkv=gqkv.data_ptr(), wo=go.data_ptr(), wgu=ggu.data_ptr(), wdown=gdown.data_ptr(),
                        attn_norm=p("attention_norm"), mlp_norm=p("mlp_norm"), attn_in_norm=p("attention_input_norm"),
                        mlp_in_norm=p("mlp_input_norm"), q_norm=p("attention.q_norm"), k_norm=p("attention.k_norm"))
        w = self._weights()
        dx = torch.empty_like(dy)
        check(self._L.olmax_block_bwd(stream_ptr(), ctypes.byref(self.c), ctypes.byref(w), ctypes.byref(g),
                                      i32(self.window), ptr(self.cos), ptr(self.sin), ptr(self._x), ptr(dy), ptr(dx),
                                      ptr(self.acts), i64(self.acts.numel()), ptr(self.tmp), i64(self.tmp.numel())))
        self.grads = {"attention.q_proj.weight": gqkv[:HD], "attention.k_proj.weight": gqkv[HD:HD + KD],
                      "attention.v_proj.weight": gqkv[HD + KD:], "attention.o_proj.weight": go,
                      "mlp.gate_proj.weight": ggu[:F], "mlp.up_proj.weight": ggu[F:], "mlp.down_proj.weight": gdown}
        self.grads.update({k + ".weight": v for k, v in gn.items()})
        return dx
