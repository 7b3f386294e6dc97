"""Thin tensor-level wrappers over the C ABI of libolmax_hip.so.

Every function takes torch CUDA(ROCm) tensors, passes raw device pointers, sizes and the
current HIP stream through ctypes, and returns freshly allocated outputs.  torch is used
only for device memory and streams; all arithmetic happens in the HIP kernels.  2-D
operands may be row-strided views (stride(1) must be 1).
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import check, f32, i32, i64, ptr, stream_ptr

BF16 = torch.bfloat16


def _L():
    return _lib.load()


def _rows2d(t: torch.Tensor) -> torch.Tensor:
    assert t.dim() == 2 and t.stride(1) == 1, "expected a row-major (possibly row-strided) 2-D tensor"
    return t


def _need_gpu(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise _lib.OlmaxHipError("olmax_amd ops run on the GPU only (got a CPU tensor); there is no CPU fallback")


# ----------------------------------------------------------------------------- GEMM / linear
def gemm(a: torch.Tensor, b: torch.Tensor, *, a_layout: int = 0, b_layout: int = 0,
         residual: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
         out_f32: bool = False) -> torch.Tensor:
    """C[M,N] = A[M,K] B[N,K]^T (+ residual).  layout 0: reduction dim contiguous
    (A stored [M,K], B stored [N,K]); layout 1: stored transposed (A [K,M], B [K,N])."""
    _need_gpu(a, b, residual, out)
    a, b = _rows2d(a), _rows2d(b)
    assert a.dtype == BF16 and b.dtype == BF16
    M, K = (a.shape if a_layout == 0 else (a.shape[1], a.shape[0]))
    N, Kb = (b.shape if b_layout == 0 else (b.shape[1], b.shape[0]))
    assert K == Kb, f"reduction dims differ: {K} vs {Kb}"
    if out is None:
        out = torch.empty(M, N, device=a.device, dtype=torch.float32 if out_f32 else BF16)
    assert out.shape == (M, N) and out.stride(1) == 1
    ldr = 0
    if residual is not None:
        residual = _rows2d(residual)
        assert residual.shape == (M, N) and residual.dtype == BF16
        ldr = residual.stride(0)
    check(_L().olmax_gemm_bf16(stream_ptr(), ptr(a), ptr(b), ptr(out), ptr(residual), i32(M), i32(N), i32(K),
                               i64(a.stride(0)), i64(b.stride(0)), i64(out.stride(0)), i64(ldr),
                               i32(a_layout), i32(b_layout), i32(1 if out.dtype == torch.float32 else 0)))
    return out


def linear_fwd(x, w, residual=None, out=None):
    """y = x W^T (+ residual); W is [out, in]  (olmax.nn.functional.linear)."""
    return gemm(x, w, residual=residual, out=out)


def linear_bwd_input(dy, w, out=None):
    """dx = dy W."""
    return gemm(dy, w, b_layout=1, out=out)


def linear_bwd_weight(dy, x, out=None, out_f32=False):
    """dW = dy^T x."""
    return gemm(dy, x, a_layout=1, b_layout=1, out=out, out_f32=out_f32)


# ----------------------------------------------------------------------------- RMSNorm
def rms_norm_fwd(x, w, eps: float, out=None):
    _need_gpu(x, w)
    x = _rows2d(x)
    if out is None:
        out = torch.empty(x.shape, device=x.device, dtype=BF16)
    check(_L().olmax_rmsnorm_fwd(stream_ptr(), ptr(x), ptr(w), ptr(out), i64(x.shape[0]), i32(x.shape[1]),
                                 i64(x.stride(0)), i64(out.stride(0)), f32(eps)))
    return out


def rms_norm_bwd(x, w, dy, eps: float, dres=None, dw: Optional[torch.Tensor] = None, out=None):
    """Returns (dx [+ dres], dw fp32).  `dw` (fp32 [d]) is accumulated into when given."""
    _need_gpu(x, w, dy)
    x, dy = _rows2d(x), _rows2d(dy)
    if out is None:
        out = torch.empty(x.shape, device=x.device, dtype=BF16)
    if dw is None and w is not None:
        dw = torch.zeros(x.shape[1], device=x.device, dtype=torch.float32)
    check(_L().olmax_rmsnorm_bwd(stream_ptr(), ptr(x), ptr(w), ptr(dy), ptr(dres), ptr(out), ptr(dw),
                                 i64(x.shape[0]), i32(x.shape[1]), i64(x.stride(0)), i64(dy.stride(0)),
                                 i64(0 if dres is None else dres.stride(0)), i64(out.stride(0)), f32(eps)))
    return out, dw


# ----------------------------------------------------------------------------- RoPE (+ head-wise QK-norm)
def rope_tables(seq_len: int, head_dim: int, theta: float, device) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos/sin [S, D/2] fp32 on the GPU (olmax.nn.rope.precompute_freqs_cis, rope.py:118-145),
    computed by the library in fp32 throughout, as the reference does."""
    device = torch.device(device)
    if device.type != "cuda":
        raise _lib.OlmaxHipError("olmax_amd ops run on the GPU only; there is no CPU fallback")
    cos = torch.empty(seq_len, head_dim // 2, device=device, dtype=torch.float32)
    sin = torch.empty_like(cos)
    check(_L().olmax_rope_tables(stream_ptr(), ptr(cos), ptr(sin), i32(seq_len), i32(head_dim), f32(theta)))
    return cos, sin


def qk_rope_fwd(x, cos, sin, *, heads: int, head_dim: int, seq_len: int, w=None, eps: float = 1e-6, out=None):
    """x: [tokens, >= heads*head_dim] view.  y = rope(headwise_rmsnorm(x, w)) (norm skipped if w is None)."""
    _need_gpu(x, cos, sin, w)
    x = _rows2d(x)
    if out is None:
        out = torch.empty(x.shape[0], heads * head_dim, device=x.device, dtype=BF16)
    check(_L().olmax_qk_rope_fwd(stream_ptr(), ptr(x), ptr(out), ptr(w), ptr(cos), ptr(sin), i64(x.shape[0]),
                                 i32(heads), i32(head_dim), i32(seq_len), i64(x.stride(0)), i64(out.stride(0)), f32(eps)))
    return out


def qk_rope_bwd(dy, cos, sin, *, heads: int, head_dim: int, seq_len: int, x=None, w=None, dw=None,
                eps: float = 1e-6, out=None):
    _need_gpu(dy, cos, sin)
    dy = _rows2d(dy)
    if out is None:
        out = torch.empty(dy.shape[0], heads * head_dim, device=dy.device, dtype=BF16)
    if w is not None and dw is None:
        dw = torch.zeros(head_dim, device=dy.device, dtype=torch.float32)
    check(_L().olmax_qk_rope_bwd(stream_ptr(), ptr(dy), ptr(out), ptr(x), ptr(w), ptr(dw), ptr(cos), ptr(sin),
                                 i64(dy.shape[0]), i32(heads), i32(head_dim), i32(seq_len), i64(dy.stride(0)),
                                 i64(out.stride(0)), i64(0 if x is None else x.stride(0)), f32(eps)))
    return out, dw


# ----------------------------------------------------------------------------- gated MLP activation
_ACT = {"silu": 0, "gelu": 1}


def glu_fwd(gate, up, act: str = "silu", out=None):
    _need_gpu(gate, up)
    gate, up = _rows2d(gate), _rows2d(up)
    T, F = gate.shape
    if out is None:
        out = torch.empty(T, F, device=gate.device, dtype=BF16)
    check(_L().olmax_glu_fwd(stream_ptr(), ptr(gate), ptr(up), ptr(out), i64(T), i32(F), i64(gate.stride(0)),
                             i64(up.stride(0)), i64(out.stride(0)), i32(_ACT[act])))
    return out


def gated_mlp_in(x, w_gate_up, act: str = "silu", gate_up_out=None, save_gate_up: bool = True, out=None):
    """GatedMLP.forward up to the down projection (reference src/olmax/nn/mlp.py:69-73):
    act(x Wgate^T) * (x Wup^T) with the activation fused into the GEMM epilogue.
    w_gate_up = [Wgate; Wup] ([2F, d]).  Returns (act_out [T, F], gate|up [T, 2F] or None)."""
    _need_gpu(x, w_gate_up)
    x = _rows2d(x)
    T, d = x.shape
    F = w_gate_up.shape[0] // 2
    if out is None:
        out = torch.empty(T, F, device=x.device, dtype=BF16)
    fits = T % 256 == 0 and F % 128 == 0 and d % 64 == 0 and (T // 256) * (F // 128) >= 128
    if gate_up_out is None and (save_gate_up or not fits):
        gate_up_out = torch.empty(T, 2 * F, device=x.device, dtype=BF16)
    check(_L().olmax_gemm_glu_bf16(stream_ptr(), ptr(x), ptr(w_gate_up), ptr(gate_up_out), ptr(out), i32(T), i32(F),
                                   i32(d), i64(x.stride(0)), i64(w_gate_up.stride(0)),
                                   i64(0 if gate_up_out is None else gate_up_out.stride(0)), i64(out.stride(0)),
                                   i32(_ACT[act])))
    return out, gate_up_out


def gated_mlp_in_bwd(x, w_gate_up, dact, act: str = "silu"):
    """The gated projection re-run in a backward pass that kept nothing: from x, [Wgate; Wup] and
    dact = d loss / d(act(gate) * up) returns (act_out [T, F], d gate | d up [T, 2F]); gate | up are
    never written.  Equals gated_mlp_in followed by glu_bwd."""
    _need_gpu(x, w_gate_up, dact)
    x, dact = _rows2d(x), _rows2d(dact)
    T, d = x.shape
    F = w_gate_up.shape[0] // 2
    assert dact.shape == (T, F) and dact.dtype == BF16
    out = torch.empty(T, F, device=x.device, dtype=BF16)
    dgu = torch.empty(T, 2 * F, device=x.device, dtype=BF16)
    check(_L().olmax_gemm_glu_bwd_bf16(stream_ptr(), ptr(x), ptr(w_gate_up), ptr(dact), ptr(out), ptr(dgu), i32(T), i32(F),
                                       i32(d), i64(x.stride(0)), i64(w_gate_up.stride(0)), i64(dact.stride(0)),
                                       i64(out.stride(0)), i64(dgu.stride(0)), i32(_ACT[act])))
    return out, dgu


def qkv_rope_proj(x, w_qkv, cos, sin, *, rope_heads: int, seq_len: int, out=None):
    """q|k|v projection with RoPE applied to the first `rope_heads` heads (q then k, head_dim 128)
    in the GEMM epilogue (reference src/olmax/nn/attention.py:270-274, 298-300).  Returns [T, N]."""
    _need_gpu(x, w_qkv, cos, sin)
    x = _rows2d(x)
    T, d = x.shape
    N = w_qkv.shape[0]
    if out is None:
        out = torch.empty(T, N, device=x.device, dtype=BF16)
    check(_L().olmax_gemm_rope_bf16(stream_ptr(), ptr(x), ptr(w_qkv), ptr(out), i32(T), i32(N), i32(d), i64(x.stride(0)),
                                    i64(w_qkv.stride(0)), i64(out.stride(0)), ptr(cos), ptr(sin), i32(seq_len),
                                    i32(rope_heads)))
    return out


def glu_bwd(gate, up, dh, act: str = "silu", dgate=None, dup=None):
    _need_gpu(gate, up, dh)
    gate, up, dh = _rows2d(gate), _rows2d(up), _rows2d(dh)
    T, F = gate.shape
    if dgate is None:
        dgate = torch.empty(T, F, device=gate.device, dtype=BF16)
    if dup is None:
        dup = torch.empty(T, F, device=gate.device, dtype=BF16)
    check(_L().olmax_glu_bwd(stream_ptr(), ptr(gate), ptr(up), ptr(dh), ptr(dgate), ptr(dup), i64(T), i32(F),
                             i64(gate.stride(0)), i64(up.stride(0)), i64(dh.stride(0)), i64(dgate.stride(0)),
                             i64(dup.stride(0)), i32(_ACT[act])))
    return dgate, dup


# ----------------------------------------------------------------------------- attention
def attn_fwd(q, k, v, *, B: int, S: int, H: int, KH: int, D: int, window: Optional[int] = None,
             softcap: float = 0.0, out=None):
    """q [B*S, H*D], k/v [B*S, KH*D] (row-strided views allowed) -> (o [B*S, H*D], lse [B,H,S])."""
    _need_gpu(q, k, v)
    q, k, v = _rows2d(q), _rows2d(k), _rows2d(v)
    if out is None:
        out = torch.empty(B * S, H * D, device=q.device, dtype=BF16)
    lse = torch.empty(B, H, S, device=q.device, dtype=torch.float32)
    check(_L().olmax_attn_fwd(stream_ptr(), ptr(q), ptr(k), ptr(v), ptr(out), ptr(lse), i32(B), i32(S), i32(H),
                              i32(KH), i32(D), i64(q.stride(0)), i64(k.stride(0)), i64(v.stride(0)),
                              i64(out.stride(0)), i32(-1 if window is None else window), f32(softcap)))
    return out, lse


def attn_bwd(q, k, v, o, lse, do, *, B: int, S: int, H: int, KH: int, D: int, window: Optional[int] = None,
             softcap: float = 0.0, dq=None, dk=None, dv=None):
    _need_gpu(q, k, v, o, lse, do)
    L = _L()
    L.olmax_attn_bwd_workspace_bytes.restype = i64
    nbytes = L.olmax_attn_bwd_workspace_bytes(i32(B), i32(S), i32(H), i32(KH), i32(D))
    ws = torch.empty(nbytes, device=q.device, dtype=torch.uint8)
    if dq is None:
        dq = torch.empty(B * S, H * D, device=q.device, dtype=BF16)
    if dk is None:
        dk = torch.empty(B * S, KH * D, device=q.device, dtype=BF16)
    if dv is None:
        dv = torch.empty(B * S, KH * D, device=q.device, dtype=BF16)
    check(L.olmax_attn_bwd(stream_ptr(), ptr(q), ptr(k), ptr(v), ptr(o), ptr(lse), ptr(do), ptr(dq), ptr(dk), ptr(dv),
                           ptr(ws), i64(nbytes), i32(B), i32(S), i32(H), i32(KH), i32(D), i64(q.stride(0)),
                           i64(k.stride(0)), i64(v.stride(0)), i64(o.stride(0)), i64(do.stride(0)),
                           i64(dq.stride(0)), i64(dk.stride(0)), i64(dv.stride(0)),
                           i32(-1 if window is None else window), f32(softcap)))
    return dq, dk, dv


# ----------------------------------------------------------------------------- cross entropy / LM head
def cross_entropy(logits, labels, *, ignore_index: int = -100, softcap: float = 0.0, want_grad: bool = True,
                  inplace: bool = False, dloss: float = 1.0, reduction: str = "mean", dloss_rows=None):
    """logits [T, V] bf16 or fp32, labels [T] int32 -> (loss, dlogits or None, lse [T]);
    reduction "mean" | "sum" | "none" as cross_entropy_loss (src/olmax/nn/functional.py:70-91):
    loss is a scalar tensor, or [T] for "none" (whose per-row cotangent is dloss * dloss_rows)."""
    _need_gpu(logits, labels, dloss_rows)
    logits = _rows2d(logits)
    assert labels.dtype == torch.int32
    red = {"mean": 0, "sum": 1, "none": 2}[reduction]
    T, V = logits.shape
    L = _L()
    L.olmax_cross_entropy_workspace_bytes.restype = i64
    nbytes = L.olmax_cross_entropy_workspace_bytes(i64(T))
    ws = torch.empty(nbytes, device=logits.device, dtype=torch.uint8)
    loss = torch.empty((T,) if red == 2 else (), device=logits.device, dtype=torch.float32)
    lse = torch.empty(T, device=logits.device, dtype=torch.float32)
    d = None
    if want_grad:
        d = logits if inplace else torch.empty_like(logits)
    if dloss_rows is not None:
        assert dloss_rows.dtype == torch.float32 and dloss_rows.numel() == T and dloss_rows.is_contiguous()
    check(L.olmax_cross_entropy_reduce(stream_ptr(), ptr(logits), ptr(d), ptr(labels), ptr(loss), ptr(lse), ptr(dloss_rows),
                                       ptr(ws), i64(nbytes), i64(T), i32(V), i64(logits.stride(0)),
                                       i64(0 if d is None else d.stride(0)), i32(1 if logits.dtype == torch.float32 else 0),
                                       i32(ignore_index), f32(softcap), f32(dloss), i32(red)))
    return loss, d, lse


def lmhead_ce(h, W, labels, *, softcap: float = 0.0, ignore_index: int = -100, want_dh: bool = True,
              want_dw: bool = True, dw_f32: bool = False, dW=None, dh=None):
    """Fused LM head + CE forward/backward: returns (loss, dh, dW)."""
    _need_gpu(h, W, labels)
    assert h.is_contiguous() and W.is_contiguous() and labels.dtype == torch.int32
    T, d = h.shape
    V = W.shape[0]
    L = _L()
    L.olmax_lmhead_ce_workspace_bytes.restype = i64
    nbytes = L.olmax_lmhead_ce_workspace_bytes(i64(T), i32(V))
    ws = torch.empty(nbytes, device=h.device, dtype=torch.uint8)
    loss = torch.empty((), device=h.device, dtype=torch.float32)
    if want_dh and dh is None:
        dh = torch.empty(T, d, device=h.device, dtype=BF16)
    if want_dw and dW is None:
        dW = torch.empty(V, d, device=h.device, dtype=torch.float32 if dw_f32 else BF16)
    check(L.olmax_lmhead_ce(stream_ptr(), ptr(h), ptr(W), ptr(labels), ptr(loss), ptr(dh), ptr(dW), ptr(ws),
                            i64(nbytes), i64(T), i32(d), i32(V), i32(ignore_index), f32(softcap),
                            i32(1 if (dW is not None and dW.dtype == torch.float32) else 0)))
    return loss, dh, dW


# ----------------------------------------------------------------------------- embedding
def embed_fwd(ids, W, out=None):
    _need_gpu(ids, W)
    assert ids.dtype == torch.int32 and W.is_contiguous()
    T = ids.numel()
    V, d = W.shape
    if out is None:
        out = torch.empty(T, d, device=W.device, dtype=BF16)
    check(_L().olmax_embed_fwd(stream_ptr(), ptr(ids), ptr(W), ptr(out), i64(T), i32(d), i32(V)))
    return out


def embed_bwd(ids, dh, vocab: int, dW: Optional[torch.Tensor] = None):
    """dW (fp32 [V, d]) += scatter_add(dh by ids); allocated zeroed when not given."""
    _need_gpu(ids, dh)
    assert ids.dtype == torch.int32 and dh.is_contiguous()
    T, d = dh.shape
    if dW is None:
        dW = torch.zeros(vocab, d, device=dh.device, dtype=torch.float32)
    check(_L().olmax_embed_bwd(stream_ptr(), ptr(ids), ptr(dh), ptr(dW), i64(T), i32(d), i32(vocab)))
    return dW


# ----------------------------------------------------------------------------- optimizer
def adamw_(p, g, m, v, *, step: int, lr: float, b1: float = 0.9, b2: float = 0.999, eps: float = 1e-8,
           wd: float = 1e-4, shadow: Optional[torch.Tensor] = None, grad_scale: float = 1.0):
    """In-place fused AdamW on fp32 p/m/v; g bf16 or fp32; optional bf16 copy of the new p."""
    _need_gpu(p, g, m, v, shadow)
    assert p.dtype == m.dtype == v.dtype == torch.float32 and p.is_contiguous()
    check(_L().olmax_adamw(stream_ptr(), ptr(p), ptr(g), ptr(m), ptr(v), ptr(shadow), i64(p.numel()),
                           i32(1 if g.dtype == BF16 else 0), f32(lr), f32(b1), f32(b2), f32(eps), f32(wd),
                           i64(step), f32(grad_scale)))


def sumsq(g, out: Optional[torch.Tensor] = None):
    _need_gpu(g)
    if out is None:
        out = torch.zeros((), device=g.device, dtype=torch.float32)
    check(_L().olmax_sumsq(stream_ptr(), ptr(g), i64(g.numel()), i32(1 if g.dtype == BF16 else 0), ptr(out)))
    return out
