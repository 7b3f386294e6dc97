// Host-side orchestration of the hot path: one transformer block (three residual orderings),
// the full model loss + gradients with optional full-block activation checkpointing, and the
// fused AdamW step over every parameter leaf.  Only enqueues kernels of this library on the
// caller's stream; all memory comes from caller-provided buffers.
//
// Reference: TransformerLayer / ReorderedNormTransformerLayer / GemmaTransformerLayer
// (src/olmax/nn/transformer/layer.py:80-94, 102-116, 169-185), Transformer.forward
// (src/olmax/nn/transformer/model.py:95-136), compute_loss_and_grads and step_optimizer
// (src/olmax/train/trainer.py:723-757).  The backward pass, which the reference obtains from
// eqx.filter_value_and_grad, is written out by hand here.
#include "common.h"
#include "olmax_hip.h"

namespace {

struct Dims {
  int64_t T;
  int d, H, K, D, F, HD, KD, QKV, B, S;
};
Dims dims_of(const olmax_model_config* c) {
  Dims m;
  m.B = c->batch;
  m.S = c->seq_len;
  m.T = (int64_t)c->batch * c->seq_len;
  m.d = c->d_model;
  m.H = c->n_heads;
  m.K = c->n_kv_heads;
  m.D = c->head_dim;
  m.F = c->hidden;
  m.HD = m.H * m.D;
  m.KD = m.K * m.D;
  m.QKV = m.HD + 2 * m.KD;
  return m;
}

int check_cfg(const olmax_model_config* c) {
  OLMAX_CHECK(c, OLMAX_ERR_ARG, "model config is null");
  OLMAX_CHECK(c->vocab > 0 && c->d_model > 0 && c->n_layers >= 0 && c->n_heads > 0 && c->n_kv_heads > 0 &&
                  c->head_dim > 0 && c->hidden > 0 && c->batch > 0 && c->seq_len > 0,
              OLMAX_ERR_SHAPE, "model config: sizes must be positive");
  OLMAX_CHECK(c->n_heads % c->n_kv_heads == 0, OLMAX_ERR_SHAPE, "model config: n_heads must be a multiple of n_kv_heads");
  OLMAX_CHECK(c->layer_type >= 0 && c->layer_type <= 2 && (c->act == 0 || c->act == 1), OLMAX_ERR_ARG, "model config: bad layer_type/act");
  OLMAX_CHECK(c->qk_norm >= 0 && c->qk_norm <= 2, OLMAX_ERR_ARG, "model config: qk_norm must be 0 (off), 1 (head-wise) or 2 (full width)");
  OLMAX_CHECK(c->head_dim % 2 == 0, OLMAX_ERR_SHAPE, "model config: head_dim must be even");
  OLMAX_CHECK(c->d_model % 8 == 0 && c->hidden % 8 == 0 && c->head_dim % 8 == 0, OLMAX_ERR_SHAPE,
              "model config: d_model, hidden and head_dim must be multiples of 8 (128-bit rows)");
  return OLMAX_OK;
}

struct Arena {
  char* base;
  int64_t off = 0;
  explicit Arena(void* b) : base((char*)b) {}
  template <typename T>
  T* take(int64_t n) {
    T* p = base ? (T*)(base + off) : nullptr;
    off += ((n * (int64_t)sizeof(T) + 255) / 256) * 256;
    return p;
  }
};

struct Acts {
  bf16 *xn, *qkv, *qkr, *o;
  float* lse;
  bf16 *a_out, *h, *hn, *gu, *act, *m_out;
};
Acts carve_acts(const olmax_model_config* c, Arena& a) {
  const Dims m = dims_of(c);
  Acts s{};
  const int lt = c->layer_type;
  if (lt != 1) s.xn = a.take<bf16>(m.T * m.d);
  s.qkv = a.take<bf16>(m.T * m.QKV);
  if (c->qk_norm) s.qkr = a.take<bf16>(m.T * (m.HD + m.KD));
  s.o = a.take<bf16>(m.T * m.HD);
  s.lse = a.take<float>((int64_t)m.B * m.H * m.S);
  if (lt != 0) s.a_out = a.take<bf16>(m.T * m.d);
  s.h = a.take<bf16>(m.T * m.d);
  if (lt != 1) s.hn = a.take<bf16>(m.T * m.d);
  s.gu = a.take<bf16>(m.T * 2 * m.F);
  s.act = a.take<bf16>(m.T * m.F);
  if (lt != 0) s.m_out = a.take<bf16>(m.T * m.d);
  return s;
}

struct Tmp {
  bf16 *dact, *dgu, *d1, *d2, *d_o, *dqkv, *dqkr;
  void* attn_ws;
  int64_t attn_ws_bytes;
};
Tmp carve_tmp(const olmax_model_config* c, Arena& a) {
  const Dims m = dims_of(c);
  Tmp t{};
  t.dact = a.take<bf16>(m.T * m.F);
  t.dgu = a.take<bf16>(m.T * 2 * m.F);
  t.d1 = a.take<bf16>(m.T * m.d);
  t.d2 = a.take<bf16>(m.T * m.d);
  t.d_o = a.take<bf16>(m.T * m.HD);
  t.dqkv = a.take<bf16>(m.T * m.QKV);
  if (c->qk_norm) t.dqkr = a.take<bf16>(m.T * (m.HD + m.KD));
  // every buffer of the arena is 256-byte aligned and every row stride a multiple of 8, so head
  // dim 128 always takes the MFMA path, which needs delta only (the generic path's two fp32
  // accumulators would be 256 MiB at the 7B shape)
  t.attn_ws_bytes = m.D == 128 ? olmax_attn_bwd_workspace_bytes_aligned(m.B, m.S, m.H)
                               : olmax_attn_bwd_workspace_bytes(m.B, m.S, m.H, m.K, m.D);
  t.attn_ws = a.take<char>(t.attn_ws_bytes);
  return t;
}

#define RC(x)            \
  do {                   \
    int rc__ = (x);      \
    if (rc__) return rc__; \
  } while (0)

// y[T,out] = x[T,in] W[out,in]^T (+ res)
int lin_fwd(hipStream_t s, const bf16* x, int64_t ldx, const void* W, int in, int out, bf16* y, int64_t ldy,
            const bf16* res, int64_t ldres, int64_t T) {
  return olmax_gemm_bf16(s, x, W, y, res, (int)T, out, in, ldx, in, ldy, ldres, 0, 0, 0);
}
// dx[T,in] = dy[T,out] W[out,in] (+ res)
int lin_dx(hipStream_t s, const bf16* dy, int64_t lddy, const void* W, int in, int out, bf16* dx, int64_t lddx,
           const bf16* res, int64_t ldres, int64_t T) {
  return olmax_gemm_bf16(s, dy, W, dx, res, (int)T, in, out, lddy, in, lddx, ldres, 0, 1, 0);
}
// dW[out,in] = dy[T,out]^T x[T,in]
int lin_dw(hipStream_t s, const bf16* dy, int64_t lddy, const bf16* x, int64_t ldx, int in, int out, void* dW,
           int64_t T, int out_f32 = 0) {
  return olmax_gemm_bf16(s, dy, x, dW, nullptr, out, in, (int)T, lddy, ldx, in, 0, 1, 1, out_f32);
}

// need_y == false (recompute before the backward): the block output itself is not an input of
// the backward pass, so the GEMM / norm that only produces it is skipped.
// Points inside a block's backward pass at which the overlapped train step may start queued
// optimizer work on its second stream (set only while olmax_model_train_step runs).
enum { POINT_RECOMPUTE_ATTN = 1, POINT_ATTN_BWD = 2, POINT_AFTER_DACT = 3 };
struct StepHook {
  int (*fn)(void* ctx, int point) = nullptr;
  void* ctx = nullptr;
};
thread_local StepHook g_hook;
inline int hook_point(int point) { return g_hook.fn ? g_hook.fn(g_hook.ctx, point) : OLMAX_OK; }

// defer_mlp (recompute of a pre-norm block only): stop after the MLP's input norm; the gated
// projection is re-run by the backward pass itself, fused with the GLU backward
// (olmax_gemm_glu_bwd_bf16), so gate | up are never written.
int block_forward(hipStream_t s, const olmax_model_config* c, const olmax_block_weights* w, int window,
                  const float* cos_t, const float* sin_t, const bf16* x, bf16* y, const Acts& a,
                  bool need_y = true, bool save_gu = true, bool defer_mlp = false) {
  const Dims m = dims_of(c);
  const int lt = c->layer_type;
  const float eps = c->eps;
  const bf16* attn_in = x;
  if (lt != 1) {
    RC(olmax_rmsnorm_fwd(s, x, lt == 0 ? w->attn_norm : w->attn_in_norm, a.xn, m.T, m.d, m.d, m.d, eps));
    attn_in = a.xn;
  }
  // without QK-norm the rotary embedding rides in the projection's epilogue (head_dim 128)
  const bool rope_in_gemm = !c->qk_norm && m.D == 128;
  if (rope_in_gemm)
    RC(olmax_gemm_rope_bf16(s, attn_in, w->wqkv, a.qkv, (int)m.T, m.QKV, m.d, m.d, m.d, m.QKV, cos_t, sin_t, m.S, m.H + m.K));
  else
    RC(lin_fwd(s, attn_in, m.d, w->wqkv, m.d, m.QKV, a.qkv, m.QKV, nullptr, 0, m.T));
  const bf16 *qp, *kp;
  int64_t ldqk;
  if (c->qk_norm == 2) {
    // full-width QK-norm (attention.py:281-284): one RMSNorm over all heads of q (and of k)
    // before the reshape, then the rotation of the normalised heads in place
    ldqk = m.HD + m.KD;
    RC(olmax_rmsnorm_fwd(s, a.qkv, w->q_norm, a.qkr, m.T, m.HD, m.QKV, ldqk, eps));
    RC(olmax_rmsnorm_fwd(s, a.qkv + m.HD, w->k_norm, a.qkr + m.HD, m.T, m.KD, m.QKV, ldqk, eps));
    RC(olmax_qk_rope_fwd(s, a.qkr, a.qkr, nullptr, cos_t, sin_t, m.T, m.H + m.K, m.D, m.S, ldqk, ldqk, eps));
    qp = a.qkr;
    kp = a.qkr + m.HD;
  } else if (c->qk_norm) {
    ldqk = m.HD + m.KD;
    RC(olmax_qk_rope_fwd(s, a.qkv, a.qkr, w->q_norm, cos_t, sin_t, m.T, m.H, m.D, m.S, m.QKV, ldqk, eps));
    RC(olmax_qk_rope_fwd(s, a.qkv + m.HD, a.qkr + m.HD, w->k_norm, cos_t, sin_t, m.T, m.K, m.D, m.S, m.QKV, ldqk, eps));
    qp = a.qkr;
    kp = a.qkr + m.HD;
  } else {
    ldqk = m.QKV;
    if (!rope_in_gemm) RC(olmax_qk_rope_fwd(s, a.qkv, a.qkv, nullptr, cos_t, sin_t, m.T, m.H + m.K, m.D, m.S, m.QKV, m.QKV, eps));
    qp = a.qkv;
    kp = a.qkv + m.HD;
  }
  if (!need_y) RC(hook_point(POINT_RECOMPUTE_ATTN));
  RC(olmax_attn_fwd(s, qp, kp, a.qkv + m.HD + m.KD, a.o, a.lse, m.B, m.S, m.H, m.K, m.D, ldqk, ldqk, m.QKV, m.HD,
                    window, c->attn_softcap));
  if (lt == 0) {
    RC(lin_fwd(s, a.o, m.HD, w->wo, m.HD, m.d, a.h, m.d, x, m.d, m.T));
  } else {
    RC(lin_fwd(s, a.o, m.HD, w->wo, m.HD, m.d, a.a_out, m.d, nullptr, 0, m.T));
    RC(olmax_rmsnorm_fwd_res(s, a.a_out, w->attn_norm, x, a.h, m.T, m.d, m.d, m.d, m.d, eps));
  }
  const bf16* mlp_in = a.h;
  if (lt != 1) {
    RC(olmax_rmsnorm_fwd(s, a.h, lt == 0 ? w->mlp_norm : w->mlp_in_norm, a.hn, m.T, m.d, m.d, m.d, eps));
    mlp_in = a.hn;
  }
  if (defer_mlp) return OLMAX_OK;
  // gate|up projection with the activation in the GEMM epilogue; gate|up themselves are only
  // written when a backward pass will read them (a.gu doubles as scratch for odd shapes)
  const bool fused_shape = m.T % 256 == 0 && m.F % 128 == 0 && m.d % 64 == 0 && (m.T / 256) * (m.F / 128) >= 128;
  RC(olmax_gemm_glu_bf16(s, mlp_in, w->wgu, (save_gu || !fused_shape) ? a.gu : nullptr, a.act, (int)m.T, m.F, m.d, m.d,
                         m.d, 2 * m.F, m.F, c->act));
  if (lt == 0) {
    if (need_y) RC(lin_fwd(s, a.act, m.F, w->wdown, m.F, m.d, y, m.d, a.h, m.d, m.T));
  } else {
    RC(lin_fwd(s, a.act, m.F, w->wdown, m.F, m.d, a.m_out, m.d, nullptr, 0, m.T));
    if (need_y) RC(olmax_rmsnorm_fwd_res(s, a.m_out, w->mlp_norm, a.h, y, m.T, m.d, m.d, m.d, m.d, eps));
  }
  return OLMAX_OK;
}

// attention part of the backward, shared by the three orderings:
// d_attn_out [T,d] -> gradients of wo, wqkv, q/k norms and d(attention input) into `dxin`
// (+ res_for_dx added in the projection's epilogue when given).
int attn_backward(hipStream_t s, const olmax_model_config* c, const olmax_block_weights* w,
                  const olmax_block_grads* g, int window, const float* cos_t, const float* sin_t,
                  const bf16* attn_in, const bf16* d_attn_out, bf16* dxin, const bf16* res_for_dx,
                  const Acts& a, const Tmp& t) {
  const Dims m = dims_of(c);
  const float eps = c->eps;
  RC(lin_dx(s, d_attn_out, m.d, w->wo, m.HD, m.d, t.d_o, m.HD, nullptr, 0, m.T));
  RC(lin_dw(s, d_attn_out, m.d, a.o, m.HD, m.HD, m.d, g->wo, m.T));
  const bf16* vp = a.qkv + m.HD + m.KD;
  RC(hook_point(POINT_ATTN_BWD));
  if (c->qk_norm) {
    const int64_t ldqk = m.HD + m.KD;
    RC(olmax_attn_bwd(s, a.qkr, a.qkr + m.HD, vp, a.o, a.lse, t.d_o, t.dqkr, t.dqkr + m.HD, t.dqkv + m.HD + m.KD,
                      t.attn_ws, t.attn_ws_bytes, m.B, m.S, m.H, m.K, m.D, ldqk, ldqk, m.QKV, m.HD, m.HD, ldqk, ldqk,
                      m.QKV, window, c->attn_softcap));
    if (c->qk_norm == 2) {
      RC(olmax_qk_rope_bwd(s, t.dqkr, t.dqkr, nullptr, nullptr, nullptr, cos_t, sin_t, m.T, m.H + m.K, m.D, m.S, ldqk, ldqk, 0, eps));
      RC(olmax_rmsnorm_bwd(s, a.qkv, w->q_norm, t.dqkr, nullptr, t.dqkv, g->q_norm, m.T, m.HD, m.QKV, ldqk, 0, m.QKV, eps));
      RC(olmax_rmsnorm_bwd(s, a.qkv + m.HD, w->k_norm, t.dqkr + m.HD, nullptr, t.dqkv + m.HD, g->k_norm, m.T, m.KD, m.QKV, ldqk, 0,
                           m.QKV, eps));
    } else {
      RC(olmax_qk_rope_bwd(s, t.dqkr, t.dqkv, a.qkv, w->q_norm, g->q_norm, cos_t, sin_t, m.T, m.H, m.D, m.S, ldqk, m.QKV,
                           m.QKV, eps));
      RC(olmax_qk_rope_bwd(s, t.dqkr + m.HD, t.dqkv + m.HD, a.qkv + m.HD, w->k_norm, g->k_norm, cos_t, sin_t, m.T, m.K,
                           m.D, m.S, ldqk, m.QKV, m.QKV, eps));
    }
  } else {
    RC(olmax_attn_bwd(s, a.qkv, a.qkv + m.HD, vp, a.o, a.lse, t.d_o, t.dqkv, t.dqkv + m.HD, t.dqkv + m.HD + m.KD,
                      t.attn_ws, t.attn_ws_bytes, m.B, m.S, m.H, m.K, m.D, m.QKV, m.QKV, m.QKV, m.HD, m.HD, m.QKV,
                      m.QKV, m.QKV, window, c->attn_softcap));
    RC(olmax_qk_rope_bwd(s, t.dqkv, t.dqkv, nullptr, nullptr, nullptr, cos_t, sin_t, m.T, m.H + m.K, m.D, m.S, m.QKV,
                         m.QKV, 0, eps));
  }
  RC(lin_dx(s, t.dqkv, m.QKV, w->wqkv, m.d, m.QKV, dxin, m.d, res_for_dx, m.d, m.T));
  RC(lin_dw(s, t.dqkv, m.QKV, attn_in, m.d, m.d, m.QKV, g->wqkv, m.T));
  return OLMAX_OK;
}

// MLP part: d_mlp_out [T,d] -> grads of wdown, wgu and d(mlp input) into `dxin` (+ res).
// deferred: the block's recompute stopped before the MLP and d act = d_mlp_out Wdown is already in
// t.dact; the gated projection runs here in its backward form (act for the down projection's
// weight gradient, d gate | d up straight from the accumulators).
int mlp_backward(hipStream_t s, const olmax_model_config* c, const olmax_block_weights* w,
                 const olmax_block_grads* g, const bf16* mlp_in, const bf16* d_mlp_out, bf16* dxin,
                 const bf16* res_for_dx, const Acts& a, const Tmp& t, bool deferred = false) {
  const Dims m = dims_of(c);
  if (deferred) {
    RC(olmax_gemm_glu_bwd_bf16(s, mlp_in, w->wgu, t.dact, a.act, t.dgu, (int)m.T, m.F, m.d, m.d, m.d, m.F, m.F, 2 * m.F, c->act));
  } else {
    RC(lin_dx(s, d_mlp_out, m.d, w->wdown, m.F, m.d, t.dact, m.F, nullptr, 0, m.T));
  }
  RC(lin_dw(s, d_mlp_out, m.d, a.act, m.F, m.F, m.d, g->wdown, m.T));
  if (!deferred)
    RC(olmax_glu_bwd(s, a.gu, a.gu + m.F, t.dact, t.dgu, t.dgu + m.F, m.T, m.F, 2 * m.F, 2 * m.F, m.F, 2 * m.F, 2 * m.F,
                     c->act));
  RC(lin_dx(s, t.dgu, 2 * m.F, w->wgu, m.d, 2 * m.F, dxin, m.d, res_for_dx, m.d, m.T));
  RC(lin_dw(s, t.dgu, 2 * m.F, mlp_in, m.d, m.d, 2 * m.F, g->wgu, m.T));
  return OLMAX_OK;
}

int block_backward(hipStream_t s, const olmax_model_config* c, const olmax_block_weights* w,
                   const olmax_block_grads* g, int window, const float* cos_t, const float* sin_t,
                   const bf16* x, const bf16* dy, bf16* dx, const Acts& a, const Tmp& t, bool mlp_deferred = false) {
  const Dims m = dims_of(c);
  const int lt = c->layer_type;
  const float eps = c->eps;
  if (lt == 0) {
    RC(mlp_backward(s, c, w, g, a.hn, dy, t.d1, nullptr, a, t, mlp_deferred));                         // d1 = d hn
    RC(olmax_rmsnorm_bwd(s, a.h, w->mlp_norm, t.d1, dy, t.d2, g->mlp_norm, m.T, m.d, m.d, m.d, m.d, m.d, eps));  // d2 = dh
    RC(attn_backward(s, c, w, g, window, cos_t, sin_t, a.xn, t.d2, t.d1, nullptr, a, t));              // d1 = d xn
    RC(olmax_rmsnorm_bwd(s, x, w->attn_norm, t.d1, t.d2, dx, g->attn_norm, m.T, m.d, m.d, m.d, m.d, m.d, eps));
  } else if (lt == 1) {
    RC(olmax_rmsnorm_bwd(s, a.m_out, w->mlp_norm, dy, nullptr, t.d1, g->mlp_norm, m.T, m.d, m.d, m.d, 0, m.d, eps));  // d1 = dm
    RC(mlp_backward(s, c, w, g, a.h, t.d1, t.d2, dy, a, t));                                           // d2 = dh
    RC(olmax_rmsnorm_bwd(s, a.a_out, w->attn_norm, t.d2, nullptr, t.d1, g->attn_norm, m.T, m.d, m.d, m.d, 0, m.d, eps));  // d1 = da
    RC(attn_backward(s, c, w, g, window, cos_t, sin_t, x, t.d1, dx, t.d2, a, t));
  } else {
    RC(olmax_rmsnorm_bwd(s, a.m_out, w->mlp_norm, dy, nullptr, t.d1, g->mlp_norm, m.T, m.d, m.d, m.d, 0, m.d, eps));  // d1 = dm
    // d(hn) must not overwrite dm while the weight gradient still reads it: the MLP part
    // finishes with dm before the input projection's dx is written into d2
    RC(mlp_backward(s, c, w, g, a.hn, t.d1, t.d2, nullptr, a, t));                                     // d2 = d hn
    RC(olmax_rmsnorm_bwd(s, a.h, w->mlp_in_norm, t.d2, dy, t.d1, g->mlp_in_norm, m.T, m.d, m.d, m.d, m.d, m.d, eps));  // d1 = dh
    RC(olmax_rmsnorm_bwd(s, a.a_out, w->attn_norm, t.d1, nullptr, t.d2, g->attn_norm, m.T, m.d, m.d, m.d, 0, m.d, eps));  // d2 = da
    // d(xn) goes to dx as scratch, then the final norm backward combines it with dh
    RC(attn_backward(s, c, w, g, window, cos_t, sin_t, a.xn, t.d2, t.d2, nullptr, a, t));              // d2 = d xn (in place)
    RC(olmax_rmsnorm_bwd(s, x, w->attn_in_norm, t.d2, t.d1, dx, g->attn_in_norm, m.T, m.d, m.d, m.d, m.d, m.d, eps));
  }
  return OLMAX_OK;
}

// ---- flat parameter layout ----
struct LayerOff {
  int64_t wqkv, wo, wgu, wdown, attn_norm, mlp_norm, attn_in_norm, mlp_in_norm, q_norm, k_norm;
  int64_t f_attn_norm, f_mlp_norm, f_attn_in_norm, f_mlp_in_norm, f_q_norm, f_k_norm;  // fp32 grad offsets
};
struct Layout {
  int64_t embedding, final_norm, lm_head, total;
  int64_t f_embedding, f_final_norm, f_total;
  int64_t layers_begin;
};
// Big matrices first inside each layer (so q,k,v and gate,up are adjacent), then the vectors.
void layer_offsets(const olmax_model_config* c, int l, const Layout& L, int64_t per_layer, int64_t per_layer_f,
                   LayerOff& o) {
  const Dims m = dims_of(c);
  int64_t p = L.layers_begin + (int64_t)l * per_layer;
  o.wqkv = p; p += (int64_t)m.QKV * m.d;
  o.wo = p; p += (int64_t)m.d * m.HD;
  o.wgu = p; p += (int64_t)2 * m.F * m.d;
  o.wdown = p; p += (int64_t)m.d * m.F;
  o.attn_norm = p; p += m.d;
  o.mlp_norm = p; p += m.d;
  o.attn_in_norm = o.mlp_in_norm = o.q_norm = o.k_norm = -1;
  if (c->layer_type == 2) { o.attn_in_norm = p; p += m.d; o.mlp_in_norm = p; p += m.d; }
  const int qn = c->qk_norm == 2 ? m.HD : m.D, kn = c->qk_norm == 2 ? m.KD : m.D;  // full width or per head
  if (c->qk_norm) { o.q_norm = p; p += qn; o.k_norm = p; p += kn; }
  int64_t f = L.f_embedding + (int64_t)c->vocab * m.d + (int64_t)l * per_layer_f;
  o.f_attn_norm = f; f += m.d;
  o.f_mlp_norm = f; f += m.d;
  o.f_attn_in_norm = o.f_mlp_in_norm = o.f_q_norm = o.f_k_norm = -1;
  if (c->layer_type == 2) { o.f_attn_in_norm = f; f += m.d; o.f_mlp_in_norm = f; f += m.d; }
  if (c->qk_norm) { o.f_q_norm = f; f += qn; o.f_k_norm = f; f += kn; }
}
int64_t per_layer_params(const olmax_model_config* c) {
  const Dims m = dims_of(c);
  int64_t n = (int64_t)m.QKV * m.d + (int64_t)m.d * m.HD + (int64_t)3 * m.F * m.d + 2 * m.d;
  if (c->layer_type == 2) n += 2 * m.d;
  if (c->qk_norm) n += c->qk_norm == 2 ? m.HD + m.KD : 2 * m.D;
  return n;
}
int64_t per_layer_f32(const olmax_model_config* c) {
  const Dims m = dims_of(c);
  int64_t n = 2 * m.d;
  if (c->layer_type == 2) n += 2 * m.d;
  if (c->qk_norm) n += c->qk_norm == 2 ? m.HD + m.KD : 2 * m.D;
  return n;
}
Layout layout_of(const olmax_model_config* c) {
  const Dims m = dims_of(c);
  Layout L;
  L.embedding = 0;
  L.layers_begin = (int64_t)c->vocab * m.d;
  int64_t p = L.layers_begin + (int64_t)c->n_layers * per_layer_params(c);
  L.final_norm = p; p += m.d;
  L.lm_head = -1;
  if (!c->tied) { L.lm_head = p; p += (int64_t)c->vocab * m.d; }
  L.total = p;
  L.f_embedding = 0;
  L.f_final_norm = (int64_t)c->vocab * m.d + (int64_t)c->n_layers * per_layer_f32(c);
  L.f_total = L.f_final_norm + m.d;
  return L;
}

struct ModelWs {
  bf16* xs;       // [(L+1), T, d] layer inputs (xs[L] = final hidden state)
  bf16* hn;       // [T, d] final-normed hidden
  bf16 *da, *db;  // [T, d] gradient ping-pong
  void* head_ws;
  int64_t head_ws_bytes;
  Tmp tmp;
  char* acts_base;
  int64_t acts_stride;
};
ModelWs carve_model(const olmax_model_config* c, Arena& a, bool need_bwd) {
  const Dims m = dims_of(c);
  ModelWs w{};
  w.xs = a.take<bf16>((int64_t)(c->n_layers + 1) * m.T * m.d);
  w.hn = a.take<bf16>(m.T * m.d);
  w.da = a.take<bf16>(m.T * m.d);
  w.db = a.take<bf16>(m.T * m.d);
  w.head_ws_bytes = olmax_lmhead_ce_workspace_bytes(m.T, c->vocab);
  w.head_ws = a.take<char>(w.head_ws_bytes);
  if (need_bwd) w.tmp = carve_tmp(c, a);
  Arena probe(nullptr);
  carve_acts(c, probe);
  w.acts_stride = probe.off;
  const int sets = (c->checkpoint || !need_bwd) ? 1 : c->n_layers;
  w.acts_base = a.take<char>(w.acts_stride * (sets > 0 ? sets : 1));
  return w;
}

void fill_weights(const olmax_model_config* c, const bf16* P, const LayerOff& o, olmax_block_weights& w) {
  w.wqkv = P + o.wqkv;
  w.wo = P + o.wo;
  w.wgu = P + o.wgu;
  w.wdown = P + o.wdown;
  w.attn_norm = P + o.attn_norm;
  w.mlp_norm = P + o.mlp_norm;
  w.attn_in_norm = o.attn_in_norm >= 0 ? P + o.attn_in_norm : nullptr;
  w.mlp_in_norm = o.mlp_in_norm >= 0 ? P + o.mlp_in_norm : nullptr;
  w.q_norm = o.q_norm >= 0 ? P + o.q_norm : nullptr;
  w.k_norm = o.k_norm >= 0 ? P + o.k_norm : nullptr;
}
void fill_grads(bf16* G, float* Gf, const LayerOff& o, olmax_block_grads& g) {
  g.wqkv = G + o.wqkv;
  g.wo = G + o.wo;
  g.wgu = G + o.wgu;
  g.wdown = G + o.wdown;
  g.attn_norm = Gf + o.f_attn_norm;
  g.mlp_norm = Gf + o.f_mlp_norm;
  g.attn_in_norm = o.f_attn_in_norm >= 0 ? Gf + o.f_attn_in_norm : nullptr;
  g.mlp_in_norm = o.f_mlp_in_norm >= 0 ? Gf + o.f_mlp_in_norm : nullptr;
  g.q_norm = o.f_q_norm >= 0 ? Gf + o.f_q_norm : nullptr;
  g.k_norm = o.f_k_norm >= 0 ? Gf + o.f_k_norm : nullptr;
}

// Called from model_run when every gradient of a group of leaves is final:
// layer >= 0: that layer's leaves; -1: final norm and (untied) LM head; -2: embedding.
struct GradReady {
  int (*fn)(void* ctx, int layer) = nullptr;
  void* ctx = nullptr;
  int operator()(int layer) const { return fn ? fn(ctx, layer) : OLMAX_OK; }
};

int model_run(hipStream_t s, const olmax_model_config* c, const int32_t* windows, const float* const* cos_tables,
              const float* const* sin_tables, const void* params_bf16, const int32_t* ids, const int32_t* labels,
              float* loss, void* grad_bf16, float* grad_f32, void* workspace, int64_t workspace_bytes, bool bwd,
              GradReady ready = GradReady()) {
  RC(check_cfg(c));
  OLMAX_CHECK(params_bf16 && ids && labels && loss && workspace, OLMAX_ERR_ARG, "olmax_model: null pointer");
  OLMAX_CHECK(!bwd || (grad_bf16 && grad_f32), OLMAX_ERR_ARG, "olmax_model: gradient buffers are null");
  OLMAX_CHECK(c->n_layers == 0 || (windows && cos_tables && sin_tables), OLMAX_ERR_ARG, "olmax_model: per-layer tables are null");
  OLMAX_CHECK((((uintptr_t)workspace) & 255) == 0, OLMAX_ERR_ALIGN, "olmax_model: workspace must be 256-byte aligned");
  OLMAX_CHECK(workspace_bytes >= olmax_model_workspace_bytes(c), OLMAX_ERR_WORKSPACE,
              "olmax_model: workspace needs %ld bytes", (long)olmax_model_workspace_bytes(c));
  const Dims m = dims_of(c);
  const Layout L = layout_of(c);
  const int64_t plp = per_layer_params(c), plf = per_layer_f32(c);
  const bf16* P = (const bf16*)params_bf16;
  bf16* G = (bf16*)grad_bf16;
  Arena arena(workspace);
  ModelWs w = carve_model(c, arena, true);
  const int64_t Td = m.T * m.d;
  const int nl = c->n_layers;
  const bool keep = bwd && !c->checkpoint;

  // RAII scope: a failing RC() return still closes the range
  struct Range {
    bool open = true;
    Range(const char* f, int l) { olmax_range_push(f, l); }
    void end() {
      if (open) olmax_range_pop();
      open = false;
    }
    ~Range() { end(); }
  };
  RC(olmax_embed_fwd(s, ids, P + L.embedding, w.xs, m.T, m.d, c->vocab));
  for (int l = 0; l < nl; l++) {
    Range rg("olmax.layers.%d.forward", l);
    LayerOff o;
    layer_offsets(c, l, L, plp, plf, o);
    olmax_block_weights bw;
    fill_weights(c, P, o, bw);
    Arena aa(w.acts_base + (keep ? (int64_t)l * w.acts_stride : 0));
    Acts acts = carve_acts(c, aa);
    RC(block_forward(s, c, &bw, windows[l], cos_tables[l], sin_tables[l], w.xs + (int64_t)l * Td,
                     w.xs + (int64_t)(l + 1) * Td, acts, true, keep));
  }
  Range rg_head("olmax.lm_head_and_loss", 0);
  const bf16* xl = w.xs + (int64_t)nl * Td;
  RC(olmax_rmsnorm_fwd(s, xl, P + L.final_norm, w.hn, m.T, m.d, m.d, m.d, c->eps));
  const bf16* Wout = c->tied ? P + L.embedding : P + L.lm_head;
  if (!bwd) {
    return olmax_lmhead_ce(s, w.hn, Wout, labels, loss, nullptr, nullptr, w.head_ws, w.head_ws_bytes, m.T, m.d, c->vocab,
                           -100, c->final_softcap, 0);
  }
  // fp32 gradient accumulators (norm weights, embedding) start from zero; a tied embedding's
  // accumulator (first in the buffer) is overwritten whole by the head's weight-gradient GEMM
  // before the scatter-add, so zeroing it (4.7 GB at vocab 256000 x 4608) would be wasted traffic
  {
    const int64_t skip = c->tied ? (int64_t)c->vocab * m.d : 0;
    RC(olmax_fill_zero(s, grad_f32 + L.f_embedding + skip, (L.f_total - skip) * 4));
  }
  if (c->tied) {
    // head dW is written (fp32) straight into the embedding's accumulator; the scatter-add follows
    RC(olmax_lmhead_ce(s, w.hn, Wout, labels, loss, w.da, grad_f32 + L.f_embedding, w.head_ws, w.head_ws_bytes, m.T, m.d,
                       c->vocab, -100, c->final_softcap, 1));
  } else {
    RC(olmax_lmhead_ce(s, w.hn, Wout, labels, loss, w.da, G + L.lm_head, w.head_ws, w.head_ws_bytes, m.T, m.d, c->vocab,
                       -100, c->final_softcap, 0));
  }
  RC(olmax_rmsnorm_bwd(s, xl, P + L.final_norm, w.da, nullptr, w.db, grad_f32 + L.f_final_norm, m.T, m.d, m.d, m.d, 0,
                       m.d, c->eps));
  RC(ready(-1));
  rg_head.end();
  bf16* dcur = w.db;
  bf16* dnext = w.da;
  for (int l = nl - 1; l >= 0; l--) {
    Range rg("olmax.layers.%d.backward", l);
    LayerOff o;
    layer_offsets(c, l, L, plp, plf, o);
    olmax_block_weights bw;
    fill_weights(c, P, o, bw);
    olmax_block_grads bg;
    fill_grads(G, grad_f32, o, bg);
    Arena aa(w.acts_base + (keep ? (int64_t)l * w.acts_stride : 0));
    Acts acts = carve_acts(c, aa);
    const bf16* xin = w.xs + (int64_t)l * Td;
    // Pre-norm blocks under recompute: the gradient of the activation output only needs dY and
    // Wdown, so it goes first; the recompute then stops at the MLP's input norm and the gated
    // projection runs once, in its backward form, inside the MLP's backward (no gate | up in
    // memory, no GLU backward kernel: 0.9 GB less traffic per 7B layer).
    const bool defer = !keep && c->layer_type == 0;
    if (defer) {
      RC(lin_dx(s, dcur, m.d, bw.wdown, m.F, m.d, w.tmp.dact, m.F, nullptr, 0, m.T));
      RC(hook_point(POINT_AFTER_DACT));
    }
    if (!keep) {
      // full-block recompute of everything the backward reads
      RC(block_forward(s, c, &bw, windows[l], cos_tables[l], sin_tables[l], xin, dnext, acts, false, true, defer));
    }
    RC(block_backward(s, c, &bw, &bg, windows[l], cos_tables[l], sin_tables[l], xin, dcur, dnext, acts, w.tmp, defer));
    RC(ready(l));
    bf16* t = dcur;
    dcur = dnext;
    dnext = t;
  }
  RC(olmax_embed_bwd(s, ids, dcur, grad_f32 + L.f_embedding, m.T, m.d, c->vocab));
  RC(ready(-2));
  return OLMAX_OK;
}

// AdamW over the leaves [begin, end) of a layout; runs of adjacent bf16-gradient leaves with
// the same decay become single launches.  leaf_decay (host, one entry per leaf of the layout;
// NULL: every leaf decays) is the weight-decay mask of AdamWConfig.build.
int adamw_leaves(hipStream_t s, const olmax_leaf* leaves, int begin, int end, float* master, float* mom, float* var,
                 bf16* shadow, const bf16* G, const float* grad_f32, int64_t step, float lr, float b1, float b2,
                 float eps, float wd, const int32_t* leaf_decay, const float* dscale, int grid_cap = 512,
                 const float* hyper_dev = nullptr) {
  auto decays = [&](int i) { return !leaf_decay || leaf_decay[i] != 0; };
  int i = begin;
  while (i < end) {
    const olmax_leaf& lf = leaves[i];
    const float lwd = decays(i) ? wd : 0.f;
    if (lf.grad_f32) {
      RC(olmax_adamw_grid(s, master + lf.offset, grad_f32 + lf.grad_f32_offset, mom + lf.offset, var + lf.offset,
                          shadow + lf.offset, lf.numel, 0, lr, b1, b2, eps, lwd, step, 1.f, dscale, grid_cap, hyper_dev));
      i++;
    } else {
      int64_t n = lf.numel;
      int j = i + 1;
      while (j < end && !leaves[j].grad_f32 && leaves[j].offset == lf.offset + n && decays(j) == decays(i)) {
        n += leaves[j].numel;
        j++;
      }
      RC(olmax_adamw_grid(s, master + lf.offset, G + lf.offset, mom + lf.offset, var + lf.offset, shadow + lf.offset, n, 1,
                          lr, b1, b2, eps, lwd, step, 1.f, dscale, grid_cap, hyper_dev));
      i = j;
    }
  }
  return OLMAX_OK;
}

// state of one overlapped train step: AdamW of a leaf group is launched on `opt` as soon as
// the main stream has produced its gradients
struct OverlapCtx {
  hipStream_t main, opt;
  hipEvent_t ev;
  const olmax_leaf* leaves;
  int nleaf;
  float *master, *mom, *var;
  bf16* shadow;
  const bf16* G;
  const float* grad_f32;
  int64_t step;
  float lr, b1, b2, eps, wd;
  const int32_t* leaf_decay;
  const float* hyper_dev;
  // 0: launch as soon as the gradients are final; else at that StepHook point.  Measured on
  // the 7B step: AdamW as a one-workgroup-per-CU grid of 32-register waves launched at once
  // (it then shares CUs with the next block's forward GEMMs, whose waves leave it 32 registers
  // per lane) gains 1.3 % over the sequential step; deferring it to an attention kernel (whose
  // waves fill the register file, so the two only time-slice) loses 5 %.
  int flush_point;
  int pending[4];      // leaf groups whose gradients are final but whose AdamW is not launched yet
  int npending;
  // The (untied) LM head's update is spread over the recompute windows of the layers: its
  // gradient is final first, and a window (norm .. gate/up GEMM of one layer's recompute) has
  // room beside the 202 M parameters of a layer's own update.  Launched whole at once it runs on
  // into the top layer's backward GEMMs, which lose far more to it than the forward ones.
  int head_leaf = -1;       // index of the LM head leaf, -1: none pending
  int64_t head_done = 0;    // elements of it already updated
  int head_windows = 0;     // windows still to come
  int64_t layer_numel = 0;  // parameters of one layer (the size of a window's own update)
};
// AdamW launches the last olmax_model_train_step of this host thread put on its optimizer stream
// (0: the step took the sequential branch); read back by tests through
// olmax_model_last_step_overlapped_launches
thread_local int g_overlapped_launches = 0;
int overlap_launch(OverlapCtx* x, int layer);
int overlap_flush(void* vctx, int point) {
  OverlapCtx* x = (OverlapCtx*)vctx;
  if (point != x->flush_point && point != -1) return OLMAX_OK;
  for (int i = 0; i < x->npending; i++) RC(overlap_launch(x, x->pending[i]));
  x->npending = 0;
  return OLMAX_OK;
}
int overlap_ready(void* vctx, int layer) {
  OverlapCtx* x = (OverlapCtx*)vctx;
  if (x->flush_point == 0) return overlap_launch(x, layer);
  if (x->npending == 4) RC(overlap_flush(x, -1));
  x->pending[x->npending++] = layer;
  return OLMAX_OK;
}
// AdamW on elements [x->head_done, x->head_done + n) of the LM head leaf
int overlap_head_chunk(OverlapCtx* x, int64_t n, int grid_cap) {
  const olmax_leaf& lf = x->leaves[x->head_leaf];
  n = n < lf.numel - x->head_done ? n : lf.numel - x->head_done;
  if (n <= 0) return OLMAX_OK;
  const int64_t o = lf.offset + x->head_done;
  x->head_done += n;
  const float lwd = (!x->leaf_decay || x->leaf_decay[x->head_leaf]) ? x->wd : 0.f;
  g_overlapped_launches++;
  return olmax_adamw_grid(x->opt, x->master + o, x->G + o, x->mom + o, x->var + o, x->shadow + o, n, 1, x->lr, x->b1, x->b2, x->eps,
                          lwd, x->step, 1.f, nullptr, grid_cap, x->hyper_dev);
}

int overlap_launch(OverlapCtx* x, int layer) {
  int begin = -1, end = -1;
  for (int i = 0; i < x->nleaf; i++) {
    const olmax_leaf& lf = x->leaves[i];
    const bool in = layer >= 0 ? lf.layer == layer
                   : layer == -1 ? (lf.kind == OLMAX_LEAF_FINAL_NORM || lf.kind == OLMAX_LEAF_LM_HEAD)
                                 : lf.kind == OLMAX_LEAF_EMBEDDING;
    if (in) {
      if (begin < 0) begin = i;
      end = i + 1;
    }
  }
  if (begin < 0) return OLMAX_OK;
  g_overlapped_launches++;
  if (hipEventRecord(x->ev, x->main) != hipSuccess || hipStreamWaitEvent(x->opt, x->ev, 0) != hipSuccess)
    return olmax_set_error(OLMAX_ERR_LAUNCH, "olmax_model_train_step: event record/wait failed");
  // One workgroup per CU is the grid that disturbs the GEMMs it runs beside least, but alone it only
  // reaches 3.3 TB/s against 5.2 TB/s for two per CU: the updates that start when the backward pass
  // is over (layer 0 and the embedding) have the GPU to themselves and take the fast grid.
  const int grid_cap = (layer == 0 || layer == -2) ? 512 : 256;
  if (layer == -1 && x->head_windows > 0) {
    // final norm now; of the LM head what a window holds, i.e. a layer's worth (the first window,
    // the top layer's recompute, has no layer update beside it); the rest follows in even shares
    for (int i = begin; i < end; i++) {
      if (x->leaves[i].kind == OLMAX_LEAF_LM_HEAD && !x->leaves[i].grad_f32) {
        x->head_leaf = i;
        x->head_done = 0;
      } else {
        RC(adamw_leaves(x->opt, x->leaves, i, i + 1, x->master, x->mom, x->var, x->shadow, x->G, x->grad_f32, x->step, x->lr, x->b1,
                        x->b2, x->eps, x->wd, x->leaf_decay, nullptr, grid_cap, x->hyper_dev));
      }
    }
    if (x->head_leaf < 0) return OLMAX_OK;
    x->head_windows--;
    return overlap_head_chunk(x, (x->layer_numel + 3) / 4 * 4, grid_cap);
  }
  RC(adamw_leaves(x->opt, x->leaves, begin, end, x->master, x->mom, x->var, x->shadow, x->G, x->grad_f32, x->step, x->lr,
                  x->b1, x->b2, x->eps, x->wd, x->leaf_decay, nullptr, grid_cap, x->hyper_dev));
  if (x->head_leaf >= 0 && layer >= 0) {
    const int64_t rem = x->leaves[x->head_leaf].numel - x->head_done;
    if (layer == 0 || x->head_windows <= 0) {
      RC(overlap_head_chunk(x, rem, grid_cap));  // whatever is left, with the last layer's update
    } else {
      RC(overlap_head_chunk(x, (rem / x->head_windows + 3) / 4 * 4, grid_cap));
      x->head_windows--;
    }
  }
  return OLMAX_OK;
}

__global__ void clip_scale_kernel(const float* sumsq, float max_norm, float* out) {
  // clip_grads_by_global_norm: g * max_norm / max(max_norm, ||g||); out[1] keeps the norm
  const float n = sqrtf(*sumsq);
  out[1] = n;
  out[0] = max_norm / fmaxf(max_norm, n);
}

}  // namespace

extern "C" int64_t olmax_model_num_params(const olmax_model_config* c) {
  if (check_cfg(c)) return -1;
  return layout_of(c).total;
}
extern "C" int64_t olmax_model_grad_f32_elems(const olmax_model_config* c) {
  if (check_cfg(c)) return -1;
  return layout_of(c).f_total;
}

extern "C" int32_t olmax_model_layout(const olmax_model_config* c, olmax_leaf* out, int32_t max_leaves) {
  if (check_cfg(c)) return -1;
  const Dims m = dims_of(c);
  const Layout L = layout_of(c);
  const int64_t plp = per_layer_params(c), plf = per_layer_f32(c);
  int n = 0;
  auto put = [&](int kind, int layer, int64_t off, int rows, int cols, int gf, int64_t foff) {
    if (out && n < max_leaves) {
      out[n].kind = kind; out[n].layer = layer; out[n].offset = off; out[n].numel = (int64_t)rows * cols;
      out[n].rows = rows; out[n].cols = cols; out[n].grad_f32 = gf; out[n].grad_f32_offset = foff;
    }
    n++;
  };
  put(OLMAX_LEAF_EMBEDDING, -1, L.embedding, c->vocab, m.d, 1, L.f_embedding);
  for (int l = 0; l < c->n_layers; l++) {
    LayerOff o;
    layer_offsets(c, l, L, plp, plf, o);
    put(OLMAX_LEAF_Q, l, o.wqkv, m.HD, m.d, 0, -1);
    put(OLMAX_LEAF_K, l, o.wqkv + (int64_t)m.HD * m.d, m.KD, m.d, 0, -1);
    put(OLMAX_LEAF_V, l, o.wqkv + (int64_t)(m.HD + m.KD) * m.d, m.KD, m.d, 0, -1);
    put(OLMAX_LEAF_O, l, o.wo, m.d, m.HD, 0, -1);
    put(OLMAX_LEAF_GATE, l, o.wgu, m.F, m.d, 0, -1);
    put(OLMAX_LEAF_UP, l, o.wgu + (int64_t)m.F * m.d, m.F, m.d, 0, -1);
    put(OLMAX_LEAF_DOWN, l, o.wdown, m.d, m.F, 0, -1);
    put(OLMAX_LEAF_ATTN_NORM, l, o.attn_norm, 1, m.d, 1, o.f_attn_norm);
    put(OLMAX_LEAF_MLP_NORM, l, o.mlp_norm, 1, m.d, 1, o.f_mlp_norm);
    if (c->layer_type == 2) {
      put(OLMAX_LEAF_ATTN_IN_NORM, l, o.attn_in_norm, 1, m.d, 1, o.f_attn_in_norm);
      put(OLMAX_LEAF_MLP_IN_NORM, l, o.mlp_in_norm, 1, m.d, 1, o.f_mlp_in_norm);
    }
    if (c->qk_norm) {
      put(OLMAX_LEAF_Q_NORM, l, o.q_norm, 1, c->qk_norm == 2 ? m.HD : m.D, 1, o.f_q_norm);
      put(OLMAX_LEAF_K_NORM, l, o.k_norm, 1, c->qk_norm == 2 ? m.KD : m.D, 1, o.f_k_norm);
    }
  }
  put(OLMAX_LEAF_FINAL_NORM, -1, L.final_norm, 1, m.d, 1, L.f_final_norm);
  if (!c->tied) put(OLMAX_LEAF_LM_HEAD, -1, L.lm_head, c->vocab, m.d, 0, -1);
  return n;
}

extern "C" int64_t olmax_block_acts_bytes(const olmax_model_config* c) {
  if (check_cfg(c)) return -1;
  Arena a(nullptr);
  carve_acts(c, a);
  return a.off;
}
extern "C" int64_t olmax_block_tmp_bytes(const olmax_model_config* c) {
  if (check_cfg(c)) return -1;
  Arena a(nullptr);
  carve_tmp(c, a);
  return a.off;
}
extern "C" int64_t olmax_model_workspace_bytes(const olmax_model_config* c) {
  if (check_cfg(c)) return -1;
  Arena a(nullptr);
  carve_model(c, a, true);
  return a.off;
}

extern "C" int32_t olmax_block_fwd(hipStream_t s, const olmax_model_config* c, const olmax_block_weights* w,
                                   int32_t window, const float* cos_t, const float* sin_t, const void* x, void* y,
                                   void* acts, int64_t acts_bytes) {
  RC(check_cfg(c));
  OLMAX_CHECK(w && cos_t && sin_t && x && y && acts, OLMAX_ERR_ARG, "olmax_block_fwd: null pointer");
  OLMAX_CHECK(acts_bytes >= olmax_block_acts_bytes(c) && (((uintptr_t)acts) & 255) == 0, OLMAX_ERR_WORKSPACE,
              "olmax_block_fwd: activation buffer too small or not 256-byte aligned");
  Arena a(acts);
  Acts ac = carve_acts(c, a);
  return block_forward(s, c, w, window, cos_t, sin_t, (const bf16*)x, (bf16*)y, ac);
}

extern "C" int32_t olmax_block_bwd(hipStream_t s, const olmax_model_config* c, const olmax_block_weights* w,
                                   const olmax_block_grads* g, int32_t window, const float* cos_t, const float* sin_t,
                                   const void* x, const void* dy, void* dx, void* acts, int64_t acts_bytes, void* tmp,
                                   int64_t tmp_bytes) {
  RC(check_cfg(c));
  OLMAX_CHECK(w && g && cos_t && sin_t && x && dy && dx && acts && tmp, OLMAX_ERR_ARG, "olmax_block_bwd: null pointer");
  OLMAX_CHECK(acts_bytes >= olmax_block_acts_bytes(c) && tmp_bytes >= olmax_block_tmp_bytes(c) &&
                  (((uintptr_t)acts) & 255) == 0 && (((uintptr_t)tmp) & 255) == 0,
              OLMAX_ERR_WORKSPACE, "olmax_block_bwd: workspace too small or not 256-byte aligned");
  Arena a(acts);
  Acts ac = carve_acts(c, a);
  Arena b(tmp);
  Tmp t = carve_tmp(c, b);
  return block_backward(s, c, w, g, window, cos_t, sin_t, (const bf16*)x, (const bf16*)dy, (bf16*)dx, ac, t);
}

extern "C" int32_t olmax_model_loss_and_grads(hipStream_t s, const olmax_model_config* c, const int32_t* windows,
                                              const float* const* cos_tables, const float* const* sin_tables,
                                              const void* params_bf16, const int32_t* ids, const int32_t* labels,
                                              float* loss, void* grad_bf16, float* grad_f32, void* workspace,
                                              int64_t workspace_bytes) {
  return model_run(s, c, windows, cos_tables, sin_tables, params_bf16, ids, labels, loss, grad_bf16, grad_f32, workspace,
                   workspace_bytes, true);
}
extern "C" int32_t olmax_model_loss(hipStream_t s, const olmax_model_config* c, const int32_t* windows,
                                    const float* const* cos_tables, const float* const* sin_tables,
                                    const void* params_bf16, const int32_t* ids, const int32_t* labels, float* loss,
                                    void* workspace, int64_t workspace_bytes) {
  return model_run(s, c, windows, cos_tables, sin_tables, params_bf16, ids, labels, loss, nullptr, nullptr, workspace,
                   workspace_bytes, false);
}

extern "C" int32_t olmax_model_adamw(hipStream_t s, const olmax_model_config* c, float* master, float* mom, float* var,
                                     void* params_bf16, const void* grad_bf16, const float* grad_f32, int64_t step,
                                     float lr, float b1, float b2, float eps, float wd, const int32_t* leaf_decay,
                                     float max_grad_norm, float* norm_scratch, const float* hyper_dev) {
  RC(check_cfg(c));
  OLMAX_CHECK(master && mom && var && params_bf16 && grad_bf16 && grad_f32, OLMAX_ERR_ARG, "olmax_model_adamw: null pointer");
  OLMAX_CHECK(step >= 1 || hyper_dev, OLMAX_ERR_ARG, "olmax_model_adamw: step is 1-based");
  if (hyper_dev) step = 1;  // unused by the kernels then
  OLMAX_CHECK(max_grad_norm <= 0.f || norm_scratch, OLMAX_ERR_ARG, "olmax_model_adamw: clipping needs norm_scratch");
  const int nleaf = olmax_model_layout(c, nullptr, 0);
  olmax_leaf* leaves = new olmax_leaf[nleaf];
  olmax_model_layout(c, leaves, nleaf);
  bf16* shadow = (bf16*)params_bf16;
  const bf16* G = (const bf16*)grad_bf16;
  int rc = OLMAX_OK;
  const float* dscale = nullptr;
  if (max_grad_norm > 0.f) {
    // norm_scratch[0] accumulates sum(g^2), then becomes the clip factor read by the AdamW kernels
    rc = olmax_fill_zero(s, norm_scratch, 8);
    for (int i = 0; i < nleaf && !rc; i++) {
      const olmax_leaf& lf = leaves[i];
      rc = lf.grad_f32 ? olmax_sumsq(s, grad_f32 + lf.grad_f32_offset, lf.numel, 0, norm_scratch)
                       : olmax_sumsq(s, G + lf.offset, lf.numel, 1, norm_scratch);
    }
    if (!rc) {
      hipLaunchKernelGGL(clip_scale_kernel, dim3(1), dim3(1), 0, s, norm_scratch, max_grad_norm, norm_scratch);
      dscale = norm_scratch;
    }
  }
  if (!rc) rc = adamw_leaves(s, leaves, 0, nleaf, master, mom, var, shadow, G, grad_f32, step, lr, b1, b2, eps, wd, leaf_decay, dscale, 512, hyper_dev);
  delete[] leaves;
  return rc;
}

// Gradient accumulation over micro-batches (optax.MultiSteps, reference
// src/olmax/optim/config.py:153-154): acc is an fp32 buffer in PARAMETER layout ([num_params]);
// the k-th (0-based) micro-batch's gradients enter the running mean acc += (g - acc) / (k + 1).
extern "C" int32_t olmax_model_grad_accumulate(hipStream_t s, const olmax_model_config* c, float* acc,
                                               const void* grad_bf16, const float* grad_f32, int32_t mini_step) {
  RC(check_cfg(c));
  OLMAX_CHECK(acc && grad_bf16 && grad_f32 && mini_step >= 0, OLMAX_ERR_ARG, "olmax_model_grad_accumulate: bad argument");
  const int nleaf = olmax_model_layout(c, nullptr, 0);
  olmax_leaf* leaves = new olmax_leaf[nleaf];
  olmax_model_layout(c, leaves, nleaf);
  const bf16* G = (const bf16*)grad_bf16;
  int rc = OLMAX_OK;
  int i = 0;
  while (i < nleaf && !rc) {
    const olmax_leaf& lf = leaves[i];
    if (lf.grad_f32) {
      rc = olmax_grad_accumulate(s, acc + lf.offset, grad_f32 + lf.grad_f32_offset, lf.numel, 0, mini_step);
      i++;
    } else {  // runs of adjacent bf16-gradient leaves in one launch
      int64_t n = lf.numel;
      int j = i + 1;
      while (j < nleaf && !leaves[j].grad_f32 && leaves[j].offset == lf.offset + n) n += leaves[j++].numel;
      rc = olmax_grad_accumulate(s, acc + lf.offset, G + lf.offset, n, 1, mini_step);
      i = j;
    }
  }
  delete[] leaves;
  return rc;
}

// AdamW from accumulated fp32 gradients in parameter layout (the step MultiSteps takes on its
// last micro-batch); clipping (max_grad_norm > 0) acts on the accumulated mean, as the
// reference chains it inside MultiSteps.
extern "C" int32_t olmax_model_adamw_accumulated(hipStream_t s, const olmax_model_config* c, float* master, float* mom,
                                                 float* var, void* params_bf16, const float* acc, int64_t step, float lr,
                                                 float b1, float b2, float eps, float wd, const int32_t* leaf_decay,
                                                 float max_grad_norm, float* norm_scratch, const float* hyper_dev) {
  RC(check_cfg(c));
  OLMAX_CHECK(master && mom && var && params_bf16 && acc, OLMAX_ERR_ARG, "olmax_model_adamw_accumulated: null pointer");
  OLMAX_CHECK(step >= 1 || hyper_dev, OLMAX_ERR_ARG, "olmax_model_adamw_accumulated: step is 1-based");
  if (hyper_dev) step = 1;
  OLMAX_CHECK(max_grad_norm <= 0.f || norm_scratch, OLMAX_ERR_ARG, "olmax_model_adamw_accumulated: clipping needs norm_scratch");
  const Layout L = layout_of(c);
  bf16* shadow = (bf16*)params_bf16;
  const float* dscale = nullptr;
  if (max_grad_norm > 0.f) {
    RC(olmax_fill_zero(s, norm_scratch, 8));
    RC(olmax_sumsq(s, acc, L.total, 0, norm_scratch));
    hipLaunchKernelGGL(clip_scale_kernel, dim3(1), dim3(1), 0, s, norm_scratch, max_grad_norm, norm_scratch);
    dscale = norm_scratch;
  }
  // the leaves tile the flat buffers in layout order: one launch per run of leaves with the same decay
  const int nleaf = olmax_model_layout(c, nullptr, 0);
  olmax_leaf* leaves = new olmax_leaf[nleaf];
  olmax_model_layout(c, leaves, nleaf);
  auto decays = [&](int i) { return !leaf_decay || leaf_decay[i] != 0; };
  int rc = OLMAX_OK;
  for (int i = 0; i < nleaf && !rc;) {
    int j = i + 1;
    int64_t n = leaves[i].numel;
    while (j < nleaf && decays(j) == decays(i) && leaves[j].offset == leaves[i].offset + n) n += leaves[j++].numel;
    const int64_t o = leaves[i].offset;
    rc = olmax_adamw_grid(s, master + o, acc + o, mom + o, var + o, shadow + o, n, 0, lr, b1, b2, eps, decays(i) ? wd : 0.f, step,
                          1.f, dscale, 512, hyper_dev);
    i = j;
  }
  delete[] leaves;
  return rc;
}

// One micro-batch of training: loss + gradients, then AdamW.  With a second stream and no
// gradient clipping the optimizer update of each layer (HBM-bound) runs on `opt_stream`
// concurrently with the backward pass of the layers below it (MFMA-bound); `stream` waits for
// the optimizer stream before returning control to later work.  Both streams must have the
// default priority.  opt_stream == NULL (or clipping on) gives the plain sequence.
extern "C" int32_t olmax_model_last_step_overlapped_launches(void) { return g_overlapped_launches; }

extern "C" int32_t olmax_model_train_step(hipStream_t stream, hipStream_t opt_stream, const olmax_model_config* c,
                                          const int32_t* windows, const float* const* cos_tables,
                                          const float* const* sin_tables, float* master, float* mom, float* var,
                                          void* params_bf16, const int32_t* ids, const int32_t* labels, float* loss,
                                          void* grad_bf16, float* grad_f32, void* workspace, int64_t workspace_bytes,
                                          int64_t step, float lr, float b1, float b2, float eps, float wd,
                                          const int32_t* leaf_decay, float max_grad_norm, float* norm_scratch,
                                          const float* hyper_dev) {
  RC(check_cfg(c));
  OLMAX_CHECK(master && mom && var && params_bf16 && grad_bf16 && grad_f32, OLMAX_ERR_ARG, "olmax_model_train_step: null pointer");
  OLMAX_CHECK(step >= 1 || hyper_dev, OLMAX_ERR_ARG, "olmax_model_train_step: step is 1-based");
  if (hyper_dev) step = 1;
  g_overlapped_launches = 0;
  // Without recompute the optimizer would share the GPU with the backward GEMMs only (no
  // forward GEMMs in between), which measured 4 % slower than running it afterwards.
  if (!opt_stream || opt_stream == stream || max_grad_norm > 0.f || !c->checkpoint) {
    RC(model_run(stream, c, windows, cos_tables, sin_tables, params_bf16, ids, labels, loss, grad_bf16, grad_f32, workspace,
                 workspace_bytes, true));
    return olmax_model_adamw(stream, c, master, mom, var, params_bf16, grad_bf16, grad_f32, step, lr, b1, b2, eps, wd,
                             leaf_decay, max_grad_norm, norm_scratch, hyper_dev);
  }
  // one event per thread, created on first use and kept for the life of the process
  static thread_local hipEvent_t ev = nullptr;
  if (!ev && hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess)
    return olmax_set_error(OLMAX_ERR_LAUNCH, "olmax_model_train_step: cannot create an event");
  const int nleaf = olmax_model_layout(c, nullptr, 0);
  olmax_leaf* leaves = new olmax_leaf[nleaf];
  olmax_model_layout(c, leaves, nleaf);
  OverlapCtx x{stream, opt_stream, ev, leaves, nleaf, master, mom, var, (bf16*)params_bf16, (const bf16*)grad_bf16, grad_f32,
               step, lr, b1, b2, eps, wd, leaf_decay, hyper_dev, 0, {0, 0, 0, 0}, 0};
  x.head_windows = c->n_layers;  // one recompute window per layer
  x.layer_numel = per_layer_params(c);
  // Pre-norm blocks open their backward with the d act GEMM (dY Wdown, hoisted in front of the
  // recompute): its waves fill the register file, so an update running beside it would keep
  // its workgroups off the CUs (measured: 1.9 ms instead of 0.5).  The update of the layer
  // above therefore starts right behind that GEMM, beside the recompute's forward kernels.
  if (c->layer_type == 0) x.flush_point = POINT_AFTER_DACT;
  // the optimizer stream must not run ahead of work already queued on the main stream
  int rc = OLMAX_OK;
  if (hipEventRecord(ev, stream) != hipSuccess || hipStreamWaitEvent(opt_stream, ev, 0) != hipSuccess)
    rc = olmax_set_error(OLMAX_ERR_LAUNCH, "olmax_model_train_step: event record/wait failed");
  GradReady ready;
  ready.fn = overlap_ready;
  ready.ctx = &x;
  g_hook.fn = overlap_flush;
  g_hook.ctx = &x;
  if (!rc)
    rc = model_run(stream, c, windows, cos_tables, sin_tables, params_bf16, ids, labels, loss, grad_bf16, grad_f32, workspace,
                   workspace_bytes, true, ready);
  g_hook = StepHook();
  if (!rc) rc = overlap_flush(&x, -1);
  // join: later work on `stream` (the next step) sees every updated parameter
  if (hipEventRecord(ev, opt_stream) != hipSuccess || hipStreamWaitEvent(stream, ev, 0) != hipSuccess)
    rc = rc ? rc : olmax_set_error(OLMAX_ERR_LAUNCH, "olmax_model_train_step: join failed");
  delete[] leaves;
  return rc;
}
