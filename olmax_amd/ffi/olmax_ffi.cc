// XLA-FFI adapter of libolmax_hip: one typed handler per C-ABI entry point a JAX host binds.
//
// Each handler only unpacks XLA buffers / attributes into the plain C call of
// include/olmax_hip.h and maps the int return code to an xla::ffi::Error; all arithmetic is in
// libolmax_hip.so.  Registered from Python (olmax_amd/jax_ffi.py) with
// jax.ffi.register_ffi_target(name, jax.ffi.pycapsule(symbol), platform="ROCM").
//
// Needs the XLA FFI headers that ship inside jaxlib (jax.ffi.include_dir()): olmax_amd/build.py
// compiles this file only when xla/ffi/api/ffi.h resolves, against libolmax_hip.so.
// Scratch memory is never allocated here: every op that needs a workspace gets it as an extra
// XLA result buffer whose size the Python wrapper asks the library for (<op>_workspace_bytes).
#include <hip/hip_runtime_api.h>

#include <mutex>
#include <vector>

#include "olmax_hip.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;
using Buf = ffi::AnyBuffer;
using Out = ffi::Result<ffi::AnyBuffer>;
using I32s = ffi::Span<const int32_t>;
using Stream = ffi::PlatformStream<hipStream_t>;

static ffi::Error Status(int32_t rc) {
  return rc == OLMAX_OK ? ffi::Error::Success() : ffi::Error::InvalidArgument(olmax_last_error_string());
}
static olmax_stream_t S(hipStream_t s) { return reinterpret_cast<olmax_stream_t>(s); }
static int64_t Rows(const Buf& b) {  // product of all dimensions but the last
  int64_t n = 1;
  for (size_t i = 0; i + 1 < b.dimensions().size(); i++) n *= b.dimensions()[i];
  return n;
}
static int32_t Last(const Buf& b) { return (int32_t)b.dimensions().back(); }

// ---- attention (AttentionKernel.forward, src/olmax/nn/attention.py:96-103): q [B,S,H,D], k/v [B,S,K,D]
static ffi::Error AttnFwd(hipStream_t st, Buf q, Buf k, Buf v, Out o, Out lse, int32_t window, float softcap) {
  auto d = q.dimensions();
  if (d.size() != 4 || k.dimensions().size() != 4) return ffi::Error::InvalidArgument("olmax_attn_fwd: q/k/v must be [B,S,H,D]");
  const int32_t B = d[0], Sq = d[1], H = d[2], D = d[3], K = k.dimensions()[2];
  return Status(olmax_attn_fwd(S(st), q.untyped_data(), k.untyped_data(), v.untyped_data(), o->untyped_data(),
                               (float*)lse->untyped_data(), B, Sq, H, K, D, (int64_t)H * D, (int64_t)K * D, (int64_t)K * D,
                               (int64_t)H * D, window, softcap));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(OlmaxAttnFwd, AttnFwd,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>()
                                  .Attr<int32_t>("window").Attr<float>("softcap"));

static ffi::Error AttnBwd(hipStream_t st, Buf q, Buf k, Buf v, Buf o, Buf lse, Buf d_o, Out dq, Out dk, Out dv, Out ws,
                          int32_t window, float softcap) {
  auto d = q.dimensions();
  if (d.size() != 4 || k.dimensions().size() != 4) return ffi::Error::InvalidArgument("olmax_attn_bwd: q/k/v must be [B,S,H,D]");
  const int32_t B = d[0], Sq = d[1], H = d[2], D = d[3], K = k.dimensions()[2];
  const int64_t hd = (int64_t)H * D, kd = (int64_t)K * D;
  return Status(olmax_attn_bwd(S(st), q.untyped_data(), k.untyped_data(), v.untyped_data(), o.untyped_data(),
                               (const float*)lse.untyped_data(), d_o.untyped_data(), dq->untyped_data(), dk->untyped_data(),
                               dv->untyped_data(), ws->untyped_data(), (int64_t)ws->size_bytes(), B, Sq, H, K, D, hd, kd, kd, hd,
                               hd, hd, kd, kd, window, softcap));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(OlmaxAttnBwd, AttnBwd,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>()
                                  .Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Attr<int32_t>("window").Attr<float>("softcap"));

// ---- rms_norm (src/olmax/nn/functional.py:51-67): x [..., d], w [d]
static ffi::Error RmsNormFwd(hipStream_t st, Buf x, Buf w, Out y, float eps) {
  const int32_t d = Last(x);
  return Status(olmax_rmsnorm_fwd(S(st), x.untyped_data(), w.untyped_data(), y->untyped_data(), Rows(x), d, d, d, eps));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(OlmaxRmsNormFwd, RmsNormFwd,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Attr<float>("eps"));

// dw (fp32 [d]) is accumulated into by the kernel: it is zeroed here first (fill kernel, capturable)
static ffi::Error RmsNormBwd(hipStream_t st, Buf x, Buf w, Buf dy, Out dx, Out dw, float eps) {
  const int32_t d = Last(x);
  if (int32_t rc = olmax_fill_zero(S(st), dw->untyped_data(), (int64_t)d * 4)) return Status(rc);
  return Status(olmax_rmsnorm_bwd(S(st), x.untyped_data(), w.untyped_data(), dy.untyped_data(), nullptr, dx->untyped_data(),
                                  (float*)dw->untyped_data(), Rows(x), d, d, d, 0, d, eps));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(OlmaxRmsNormBwd, RmsNormBwd,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>().Attr<float>("eps"));

// ---- linear (src/olmax/nn/functional.py:14-27) and its two transposes: C[M,N] = A B^T with
// a_layout / b_layout 1 when the operand is stored with the reduction dimension first.
static ffi::Error Gemm(hipStream_t st, Buf a, Buf b, Out c, int32_t a_layout, int32_t b_layout) {
  const int32_t M = a_layout ? Last(a) : (int32_t)Rows(a), K = a_layout ? (int32_t)Rows(a) : Last(a);
  const int32_t N = b_layout ? Last(b) : (int32_t)Rows(b);
  return Status(olmax_gemm_bf16(S(st), a.untyped_data(), b.untyped_data(), c->untyped_data(), nullptr, M, N, K, Last(a), Last(b),
                                N, 0, a_layout, b_layout, c->element_type() == ffi::DataType::F32));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(OlmaxGemm, Gemm,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Attr<int32_t>("a_layout")
                                  .Attr<int32_t>("b_layout"));

// ---- LM head + cross entropy, forward and backward in one call (lm_head.py:59-61, functional.py:70-91)
static ffi::Error LmHeadCe(hipStream_t st, Buf h, Buf w, Buf labels, Out loss, Out dh, Out dw, Out ws, float softcap) {
  return Status(olmax_lmhead_ce(S(st), h.untyped_data(), w.untyped_data(), (const int32_t*)labels.untyped_data(),
                                (float*)loss->untyped_data(), dh->untyped_data(), dw->untyped_data(), ws->untyped_data(),
                                (int64_t)ws->size_bytes(), Rows(h), Last(h), (int32_t)Rows(w), -100, softcap,
                                dw->element_type() == ffi::DataType::F32));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(OlmaxLmHeadCe, LmHeadCe,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>()
                                  .Attr<float>("softcap"));

// ---- RoPE with the optional head-wise QK-norm (RotaryPositionalEmbedding.forward, src/olmax/nn/rope.py:68-80,
// applied at src/olmax/nn/attention.py:298-300 after the norm of :293-296): x [B,S,H,D], cos/sin [S, D/2] fp32,
// w [D] (read only when use_norm != 0).
static ffi::Error QkRopeFwd(hipStream_t st, Buf x, Buf w, Buf cos, Buf sin, Out y, int32_t use_norm, float eps) {
  auto d = x.dimensions();
  if (d.size() != 4) return ffi::Error::InvalidArgument("olmax_qk_rope_fwd: x must be [B,S,H,D]");
  const int64_t tokens = d[0] * d[1];
  const int32_t Sq = (int32_t)d[1], H = (int32_t)d[2], D = (int32_t)d[3];
  if (cos.dimensions().size() != 2 || cos.dimensions()[0] < Sq || cos.dimensions()[1] * 2 != D)
    return ffi::Error::InvalidArgument("olmax_qk_rope_fwd: cos/sin must be [>= S, D/2]");
  return Status(olmax_qk_rope_fwd(S(st), x.untyped_data(), y->untyped_data(), use_norm ? w.untyped_data() : nullptr,
                                  (const float*)cos.untyped_data(), (const float*)sin.untyped_data(), tokens, H, D, Sq,
                                  (int64_t)H * D, (int64_t)H * D, eps));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(OlmaxQkRopeFwd, QkRopeFwd,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>()
                                  .Attr<int32_t>("use_norm").Attr<float>("eps"));

// dw (fp32 [D]) is accumulated into by the kernel: zeroed here first (only with use_norm)
static ffi::Error QkRopeBwd(hipStream_t st, Buf dy, Buf x, Buf w, Buf cos, Buf sin, Out dx, Out dw, int32_t use_norm,
                            float eps) {
  auto d = x.dimensions();
  if (d.size() != 4) return ffi::Error::InvalidArgument("olmax_qk_rope_bwd: x must be [B,S,H,D]");
  const int64_t tokens = d[0] * d[1];
  const int32_t Sq = (int32_t)d[1], H = (int32_t)d[2], D = (int32_t)d[3];
  const int64_t ld = (int64_t)H * D;
  if (int32_t rc = olmax_fill_zero(S(st), dw->untyped_data(), (int64_t)dw->size_bytes())) return Status(rc);
  return Status(olmax_qk_rope_bwd(S(st), dy.untyped_data(), dx->untyped_data(), use_norm ? x.untyped_data() : nullptr,
                                  use_norm ? w.untyped_data() : nullptr, use_norm ? (float*)dw->untyped_data() : nullptr,
                                  (const float*)cos.untyped_data(), (const float*)sin.untyped_data(), tokens, H, D, Sq, ld, ld,
                                  ld, eps));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(OlmaxQkRopeBwd, QkRopeBwd,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>()
                                  .Ret<Buf>().Attr<int32_t>("use_norm").Attr<float>("eps"));

// ---- gated MLP (GatedMLP.forward, src/olmax/nn/mlp.py:69-73): the gate|up projection with the activation in the
// GEMM epilogue (x [..., K], w = [Wgate; Wup] [2F, K] -> act [..., F] and gate|up [..., 2F] for the backward),
// and the elementwise backward of act(gate) * up.  act: 0 silu, 1 tanh-gelu.
static ffi::Error GemmGlu(hipStream_t st, Buf x, Buf w, Out act_out, Out gu_out, int32_t act) {
  const int32_t K = Last(x), F2 = (int32_t)Rows(w);
  if (Last(w) != K || (F2 & 1)) return ffi::Error::InvalidArgument("olmax_gemm_glu: w must be [2F, K] with K = x's last dimension");
  return Status(olmax_gemm_glu_bf16(S(st), x.untyped_data(), w.untyped_data(), gu_out->untyped_data(), act_out->untyped_data(),
                                    (int32_t)Rows(x), F2 / 2, K, K, K, F2, F2 / 2, act));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(OlmaxGemmGlu, GemmGlu,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>().Attr<int32_t>("act"));

// gu [..., 2F] (gate | up), dh [..., F] -> dgu [..., 2F] (dgate | dup)
static ffi::Error GluBwd(hipStream_t st, Buf gu, Buf dh, Out dgu, int32_t act) {
  const int32_t F = Last(dh);
  if (Last(gu) != 2 * F) return ffi::Error::InvalidArgument("olmax_glu_bwd: gu must be [..., 2F] for dh [..., F]");
  const char* g = (const char*)gu.untyped_data();
  char* dg = (char*)dgu->untyped_data();
  return Status(olmax_glu_bwd(S(st), g, g + (int64_t)F * 2, dh.untyped_data(), dg, dg + (int64_t)F * 2, Rows(dh), F, 2 * (int64_t)F,
                              2 * (int64_t)F, F, 2 * (int64_t)F, 2 * (int64_t)F, act));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(OlmaxGluBwd, GluBwd,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Attr<int32_t>("act"));

// ---- embedding (Embedding.forward, src/olmax/nn/embedding.py:30-32) and its transpose (dW fp32, zeroed here)
static ffi::Error EmbedFwd(hipStream_t st, Buf ids, Buf w, Out out) {
  if (w.dimensions().size() != 2) return ffi::Error::InvalidArgument("olmax_embed_fwd: weight must be [V, d]");
  return Status(olmax_embed_fwd(S(st), (const int32_t*)ids.untyped_data(), w.untyped_data(), out->untyped_data(),
                                (int64_t)ids.element_count(), (int32_t)w.dimensions()[1], (int32_t)w.dimensions()[0]));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(OlmaxEmbedFwd, EmbedFwd, ffi::Ffi::Bind().Ctx<Stream>().Arg<Buf>().Arg<Buf>().Ret<Buf>());

static ffi::Error EmbedBwd(hipStream_t st, Buf ids, Buf dh, Out dw) {
  if (dw->dimensions().size() != 2) return ffi::Error::InvalidArgument("olmax_embed_bwd: dW must be [V, d]");
  if (int32_t rc = olmax_fill_zero(S(st), dw->untyped_data(), (int64_t)dw->size_bytes())) return Status(rc);
  return Status(olmax_embed_bwd(S(st), (const int32_t*)ids.untyped_data(), dh.untyped_data(), (float*)dw->untyped_data(),
                                (int64_t)ids.element_count(), (int32_t)dw->dimensions()[1], (int32_t)dw->dimensions()[0]));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(OlmaxEmbedBwd, EmbedBwd, ffi::Ffi::Bind().Ctx<Stream>().Arg<Buf>().Arg<Buf>().Ret<Buf>());

// ---- cross entropy on given logits (cross_entropy_loss / fused_cross_entropy_loss, src/olmax/nn/functional.py:70-121):
// forward -> loss (scalar, or [T] for reduction "none") and the log-normaliser * (label != ignore); backward ->
// dlogits from per-row cotangents (the wrapper folds 1/n of "mean" into them on the device).
static ffi::Error CrossEntropyFwd(hipStream_t st, Buf logits, Buf labels, Out loss, Out lse, Out ws, int32_t reduction,
                                  int32_t ignore_index, float softcap) {
  const int64_t T = Rows(logits);
  const int32_t V = Last(logits);
  return Status(olmax_cross_entropy_reduce(S(st), logits.untyped_data(), nullptr, (const int32_t*)labels.untyped_data(),
                                           (float*)loss->untyped_data(), (float*)lse->untyped_data(), nullptr, ws->untyped_data(),
                                           (int64_t)ws->size_bytes(), T, V, V, V, logits.element_type() == ffi::DataType::F32,
                                           ignore_index, softcap, 1.f, reduction));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(OlmaxCrossEntropyFwd, CrossEntropyFwd,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>()
                                  .Attr<int32_t>("reduction").Attr<int32_t>("ignore_index").Attr<float>("softcap"));

static ffi::Error CrossEntropyBwd(hipStream_t st, Buf logits, Buf labels, Buf row_cotangent, Out dlogits, Out row_loss, Out ws,
                                  int32_t ignore_index, float softcap) {
  const int64_t T = Rows(logits);
  const int32_t V = Last(logits);
  if ((int64_t)row_cotangent.element_count() != T) return ffi::Error::InvalidArgument("olmax_cross_entropy_bwd: one cotangent per row");
  return Status(olmax_cross_entropy_reduce(S(st), logits.untyped_data(), dlogits->untyped_data(), (const int32_t*)labels.untyped_data(),
                                           (float*)row_loss->untyped_data(), nullptr, (const float*)row_cotangent.untyped_data(),
                                           ws->untyped_data(), (int64_t)ws->size_bytes(), T, V, V, V,
                                           logits.element_type() == ffi::DataType::F32, ignore_index, softcap, 1.f, 2));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(OlmaxCrossEntropyBwd, CrossEntropyBwd,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>()
                                  .Attr<int32_t>("ignore_index").Attr<float>("softcap"));

// ---- AdamW on one leaf (optax.adamw as built at src/olmax/optim/config.py:136-156).  p, m, v are
// updated in place: the wrapper aliases results 0-2 to arguments 0, 2, 3 (donated buffers).
// hyper: fp32 [3] = {lr, 1 - b1^t, 1 - b2^t}, computed on the device by the caller from optax's
// count and injected learning rate, so the step count never has to reach the host.
static ffi::Error AdamW(hipStream_t st, Buf p, Buf g, Buf m, Buf v, Buf hyper, Out p_out, Out m_out, Out v_out, float b1,
                        float b2, float eps, float wd) {
  if (p_out->untyped_data() != p.untyped_data() || m_out->untyped_data() != m.untyped_data() ||
      v_out->untyped_data() != v.untyped_data())
    return ffi::Error::InvalidArgument("olmax_adamw: p, m, v must be donated (input_output_aliases {0:0, 2:1, 3:2})");
  return Status(olmax_adamw_dev(S(st), (float*)p.untyped_data(), g.untyped_data(), (float*)m.untyped_data(),
                                (float*)v.untyped_data(), nullptr, (int64_t)p.element_count(),
                                g.element_type() == ffi::DataType::BF16, b1, b2, eps, wd, (const float*)hyper.untyped_data(),
                                nullptr));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(OlmaxAdamW, AdamW,
                              ffi::Ffi::Bind().Ctx<Stream>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Ret<Buf>().Ret<Buf>()
                                  .Ret<Buf>().Attr<float>("b1").Attr<float>("b2").Attr<float>("eps").Attr<float>("wd"));

// ---- the whole micro-batch step (process_microbatch, src/olmax/train/trainer.py:759-777) on the flat
// buffers olmax_model_layout describes.  Arguments: master, m, v (fp32 [N]), params (bf16 [N]), ids,
// labels (int32 [B*S]), rope tables cos/sin (fp32 [n_tables, S, D/2]), hyper (fp32 [3] = {lr,
// 1 - b1^t, 1 - b2^t}: the schedule and the step count stay on the device).  Results: the four state
// buffers again (aliased to arguments 0-3: donated), loss (fp32 []), grad_bf16 (bf16 [N]),
// grad_f32 (fp32 [olmax_model_grad_f32_elems]), workspace (u8 [olmax_model_workspace_bytes]),
// norm (fp32 [2]: clip factor, gradient norm).  Attributes: `config` = the 14 integers of
// olmax_model_config in declaration order, eps / soft-caps, per-layer `windows` and `table_index`
// (which cos/sin table a layer uses), `leaf_decay` (empty: every leaf decays), hyper-parameters.
// overlap != 0 runs each layer's AdamW on a second stream this file creates once (default priority).
static ffi::Error TrainStep(hipStream_t st, Buf master, Buf m, Buf v, Buf params, Buf ids, Buf labels, Buf cos, Buf sin,
                            Buf hyper, Out master_o, Out m_o, Out v_o, Out params_o, Out loss, Out grad_bf16, Out grad_f32, Out ws, Out norm,
                            I32s config, float eps, float attn_softcap, float final_softcap, I32s windows, I32s table_index,
                            I32s leaf_decay, float b1, float b2, float adam_eps, float wd, float max_grad_norm,
                            int32_t overlap) {
  if (config.size() != 14) return ffi::Error::InvalidArgument("olmax_train_step: config must hold 14 integers");
  if (master_o->untyped_data() != master.untyped_data() || m_o->untyped_data() != m.untyped_data() ||
      v_o->untyped_data() != v.untyped_data() || params_o->untyped_data() != params.untyped_data())
    return ffi::Error::InvalidArgument("olmax_train_step: master, m, v, params must be donated (aliases {0:0, 1:1, 2:2, 3:3})");
  olmax_model_config c;
  int32_t* ci = &c.vocab;  // the 14 leading int32 fields are contiguous
  for (int i = 0; i < 14; i++) ci[i] = config[i];
  c.eps = eps; c.attn_softcap = attn_softcap; c.final_softcap = final_softcap;
  if ((int)windows.size() != c.n_layers || (int)table_index.size() != c.n_layers)
    return ffi::Error::InvalidArgument("olmax_train_step: windows / table_index need one entry per layer");
  // every attribute and buffer size is checked against what the library will read before anything is launched
  const int64_t n_params = olmax_model_num_params(&c);
  if (n_params < 0) return ffi::Error::InvalidArgument(olmax_last_error_string());
  const int32_t n_leaf = olmax_model_layout(&c, nullptr, 0);
  if (leaf_decay.size() != 0 && (int64_t)leaf_decay.size() != n_leaf)
    return ffi::Error::InvalidArgument("olmax_train_step: leaf_decay must be empty or hold one entry per leaf of olmax_model_layout");
  if (cos.dimensions().size() != 3 || sin.dimensions().size() != 3 || cos.dimensions()[1] != c.seq_len ||
      cos.dimensions()[2] * 2 != c.head_dim || sin.dimensions()[0] != cos.dimensions()[0] ||
      sin.dimensions()[1] != cos.dimensions()[1] || sin.dimensions()[2] != cos.dimensions()[2])
    return ffi::Error::InvalidArgument("olmax_train_step: cos / sin must be [n_tables, seq_len, head_dim / 2]");
  for (int l = 0; l < c.n_layers; l++)
    if (table_index[l] < 0 || table_index[l] >= cos.dimensions()[0])
      return ffi::Error::InvalidArgument("olmax_train_step: table_index entry outside the cos / sin tables");
  if ((int64_t)master.element_count() != n_params || (int64_t)m.element_count() != n_params ||
      (int64_t)v.element_count() != n_params || (int64_t)params.element_count() != n_params ||
      (int64_t)grad_bf16->element_count() != n_params)
    return ffi::Error::InvalidArgument("olmax_train_step: master, m, v, params and grad_bf16 must hold olmax_model_num_params elements");
  if ((int64_t)grad_f32->element_count() != olmax_model_grad_f32_elems(&c))
    return ffi::Error::InvalidArgument("olmax_train_step: grad_f32 must hold olmax_model_grad_f32_elems elements");
  if ((int64_t)ws->size_bytes() < olmax_model_workspace_bytes(&c))
    return ffi::Error::InvalidArgument("olmax_train_step: workspace smaller than olmax_model_workspace_bytes");
  const int64_t T = (int64_t)c.batch * c.seq_len;
  if ((int64_t)ids.element_count() != T || (int64_t)labels.element_count() != T || hyper.element_count() != 3 ||
      norm->element_count() != 2)
    return ffi::Error::InvalidArgument("olmax_train_step: ids / labels need batch * seq_len entries, hyper 3, norm 2");
  const int64_t table = cos.dimensions()[1] * cos.dimensions()[2];
  std::vector<const float*> cp(c.n_layers), sp(c.n_layers);
  for (int l = 0; l < c.n_layers; l++) {
    cp[l] = (const float*)cos.untyped_data() + table_index[l] * table;
    sp[l] = (const float*)sin.untyped_data() + table_index[l] * table;
  }
  static hipStream_t opt = nullptr;
  static std::once_flag once;
  if (overlap) std::call_once(once, [] { (void)hipStreamCreateWithFlags(&opt, hipStreamNonBlocking); });
  return Status(olmax_model_train_step(
      S(st), overlap ? S(opt) : nullptr, &c, windows.begin(), cp.data(), sp.data(), (float*)master.untyped_data(),
      (float*)m.untyped_data(), (float*)v.untyped_data(), params.untyped_data(), (const int32_t*)ids.untyped_data(),
      (const int32_t*)labels.untyped_data(), (float*)loss->untyped_data(), grad_bf16->untyped_data(),
      (float*)grad_f32->untyped_data(), ws->untyped_data(), (int64_t)ws->size_bytes(), /*step=*/0, /*lr=*/0.f, b1, b2, adam_eps,
      wd, leaf_decay.size() ? leaf_decay.begin() : nullptr, max_grad_norm, (float*)norm->untyped_data(),
      (const float*)hyper.untyped_data()));
}
XLA_FFI_DEFINE_HANDLER_SYMBOL(
    OlmaxTrainStep, TrainStep,
    ffi::Ffi::Bind().Ctx<Stream>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>().Arg<Buf>()
        .Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>().Ret<Buf>()
        .Attr<I32s>("config").Attr<float>("eps").Attr<float>("attn_softcap").Attr<float>("final_softcap")
        .Attr<I32s>("windows").Attr<I32s>("table_index").Attr<I32s>("leaf_decay")
        .Attr<float>("b1").Attr<float>("b2").Attr<float>("adam_eps").Attr<float>("wd").Attr<float>("max_grad_norm")
        .Attr<int32_t>("overlap"));
