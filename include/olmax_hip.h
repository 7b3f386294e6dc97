/*
 * libolmax_hip — C ABI of the MI355X (gfx950) transformer training hot path.
 *
 * The reference (epwalsh/OLMax) is pure JAX: it has no FFI boundary of its own, its kernels
 * come from XLA / cuBLASLt / cuDNN behind jax.jit.  Each entry point below replaces one of
 * those dispatches and cites the reference function whose arithmetic it implements; these
 * are the symbols a jax.ffi custom-call adapter (or any other host) binds.
 *
 * Conventions
 *  - All pointers are device pointers unless stated; the caller owns every buffer.
 *  - Work is only ENQUEUED on `stream`; no call synchronises or touches another stream.
 *  - Matrices are row-major with an explicit row stride in ELEMENTS ("ld*"); the last
 *    dimension is contiguous.  bf16 storage, fp32 accumulation and statistics.
 *  - Return 0 on success; negative on an argument error detected on the host before any
 *    launch (olmax_last_error_string() gives the thread-local message).  Nothing throws.
 *  - Compute entry points never allocate device memory and may be called from any host thread;
 *    what they keep between calls is immutable once set (kernel attributes, set once under
 *    std::call_once; the device's CU count) or per thread (the last error string, one HIP event of
 *    olmax_model_train_step).  The exceptions are the three process-wide DIAGNOSTIC switches at
 *    the end of this file (tile override, GEMM event profile, profiler ranges) and
 *    olmax_attn_bwd_noalloc, whose scratch array is shared by all calls on a GPU.
 *  - Arguments are flat lists of pointers, sizes and scalars (no parameter structs except the
 *    whole-model configuration); an op that needs scratch takes `workspace` + `workspace_bytes`
 *    and has a pure `<op>_workspace_bytes` companion.
 *  - Token ids follow NumPy/JAX indexing of `weight[ids]`: a negative id counts from the end and
 *    what is still outside [0, vocab) is clamped (gather and its scatter-add transpose alike);
 *    labels outside [0, vocab) follow the reference's one-hot semantics (see olmax_cross_entropy).
 */
#ifndef OLMAX_HIP_H
#define OLMAX_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* olmax_stream_t; /* == hipStream_t */

#define OLMAX_OK 0
#define OLMAX_ERR_ARG (-1)
#define OLMAX_ERR_SHAPE (-2)
#define OLMAX_ERR_ALIGN (-3)
#define OLMAX_ERR_LAUNCH (-4)
#define OLMAX_ERR_WORKSPACE (-5)

const char* olmax_last_error_string(void);
int32_t olmax_abi_version(void);

/* ---- Linear: olmax.nn.functional.linear, src/olmax/nn/functional.py:14-27 (y = x W^T) and
 * the two products JAX autodiff derives from it (dx = dy W, dW = dy^T x).
 * C[M,N] = A B^T (+ R).  a_layout/b_layout 0: operand stored with the reduction dimension
 * contiguous (A [M,K], B [N,K]); 1: stored transposed (A [K,M], B [K,N]).
 * R (optional bf16 [M,N]) is the residual of src/olmax/nn/transformer/layer.py:86,90, `x + linear(..)`
 * on bf16 arrays: C = bf16(bf16(A B^T) + R), the product rounded to bf16 first as the reference's
 * linear output is, the sum rounded again (with out_f32 != 0: C = fp32(A B^T) + R, fp32, unrounded).
 * out_f32 != 0 writes C as fp32. */
int32_t olmax_gemm_bf16(olmax_stream_t stream, const void* A, const void* B, void* C, const void* R,
                        int32_t M, int32_t N, int32_t K, int64_t lda, int64_t ldb, int64_t ldc,
                        int64_t ldr, int32_t a_layout, int32_t b_layout, int32_t out_f32);

/* ---- RMSNorm: rms_norm, src/olmax/nn/functional.py:51-67; RMSNorm.forward,
 * src/olmax/nn/normalization.py:85-87.  w may be NULL (no scale). */
int32_t olmax_rmsnorm_fwd(olmax_stream_t stream, const void* x, const void* w, void* y, int64_t rows,
                          int32_t d, int64_t ldx, int64_t ldy, float eps);
/* y = bf16(rms_norm(x, w)) + res : post-norm residual of ReorderedNormTransformerLayer /
 * GemmaTransformerLayer, src/olmax/nn/transformer/layer.py:108,112,175,181. */
int32_t olmax_rmsnorm_fwd_res(olmax_stream_t stream, const void* x, const void* w, const void* res,
                              void* y, int64_t rows, int32_t d, int64_t ldx, int64_t ldres,
                              int64_t ldy, float eps);
/* Transpose of rms_norm.  dx = d(norm)/dx^T dy (+ dres); dw (fp32 [d], optional) is
 * ACCUMULATED into with atomics: zero it first. */
int32_t olmax_rmsnorm_bwd(olmax_stream_t stream, const void* x, const void* w, const void* dy,
                          const void* dres, void* dx, float* dw, int64_t rows, int32_t d, int64_t ldx,
                          int64_t lddy, int64_t lddres, int64_t lddx, float eps);

/* ---- RoPE (+ head-wise QK-norm): RotaryPositionalEmbedding._apply_rope,
 * src/olmax/nn/rope.py:99-115 (rotate_half, fp32), applied to q and k at
 * src/olmax/nn/attention.py:298-300 after the optional head-wise norm of :293-296.
 * x/y: [tokens, heads*head_dim] views (in place allowed); position = token % seq_len;
 * cos/sin: fp32 [seq_len, head_dim/2] (precompute_freqs_cis, rope.py:118-145).
 * w != NULL: y = rope(bf16(rms_norm_per_head(x, w))). */
/* cos/sin tables [seq_len, head_dim/2] fp32: precompute_freqs_cis, src/olmax/nn/rope.py:118-145
 * (freqs = 1 / theta^(2i/D), t = arange(seq_len), their outer product and cos/sin all in fp32,
 * rope.py:127-133; RotaryPositionalEmbedding.get_freqs_cis / warmup_cache, rope.py:82-97). */
int32_t olmax_rope_tables(olmax_stream_t stream, float* cos_t, float* sin_t, int32_t seq_len,
                          int32_t head_dim, float theta);
int32_t olmax_qk_rope_fwd(olmax_stream_t stream, const void* x, void* y, const void* w,
                          const float* cos_t, const float* sin_t, int64_t tokens, int32_t heads,
                          int32_t head_dim, int32_t seq_len, int64_t ldx, int64_t ldy, float eps);
int32_t olmax_qk_rope_bwd(olmax_stream_t stream, const void* dy, void* dx, const void* x,
                          const void* w, float* dw, const float* cos_t, const float* sin_t,
                          int64_t tokens, int32_t heads, int32_t head_dim, int32_t seq_len,
                          int64_t lddy, int64_t lddx, int64_t ldx, float eps);

/* ---- Gated MLP input projection with the activation fused into the GEMM epilogue:
 * GatedMLP.forward, src/olmax/nn/mlp.py:69-73 (gate_proj, up_proj, act(gate) * up in one call).
 * W = [Wgate; Wup] ([2F, K], row stride ldw); act_out [M, F]; gu_out ([M, 2F], optional when
 * M % 256 == 0 and F % 128 == 0 and K % 64 == 0, required as scratch otherwise) receives gate|up
 * for the backward pass.  act: 0 = silu, 1 = tanh-approximated gelu.  Results equal
 * olmax_gemm_bf16 followed by olmax_glu_fwd bit for bit. */
int32_t olmax_gemm_glu_bf16(olmax_stream_t stream, const void* X, const void* W, void* gu_out, void* act_out,
                            int32_t M, int32_t F, int32_t K, int64_t ldx, int64_t ldw, int64_t ldgu,
                            int64_t ldact, int32_t act);

/* The same projection re-run in the backward pass of a block that kept nothing (full-block recompute,
 * src/olmax/activation_checkpointing.py:71-80): from X, W and dact = d loss / d(act(gate) * up) it writes
 * act_out [M, F] (the operand of the down projection's weight gradient) and dgu_out [M, 2F] =
 * d gate | d up; gate | up stay in the accumulators.  Results equal olmax_gemm_glu_bf16 followed by
 * olmax_glu_bwd bit for bit (the path taken, through dgu_out as scratch, when the shape does not fit). */
int32_t olmax_gemm_glu_bwd_bf16(olmax_stream_t stream, const void* X, const void* W, const void* dact, void* act_out,
                                void* dgu_out, int32_t M, int32_t F, int32_t K, int64_t ldx, int64_t ldw,
                                int64_t lddact, int64_t ldact, int64_t lddgu, int32_t act);

/* ---- q|k|v projection with the rotary embedding fused into the GEMM epilogue:
 * MultiheadSelfAttention.forward, src/olmax/nn/attention.py:270-274 (projections) and :298-300
 * (RoPE on q and k, src/olmax/nn/rope.py:99-115), for recipes without QK-norm.
 * out[M, N] = X W^T with W = [Wq; Wk; Wv] ([N, K], row stride ldw); the first rope_heads heads of
 * 128 columns (q then k) leave rotated, position of row r = r % seq_len, cos/sin [seq_len, 64]
 * fp32.  Equals olmax_gemm_bf16 followed by olmax_qk_rope_fwd in place (the path taken when the
 * shape does not fit: M, N % 256, K % 64, rope_heads even, >= 128 tiles). */
int32_t olmax_gemm_rope_bf16(olmax_stream_t stream, const void* X, const void* W, void* out, int32_t M, int32_t N,
                             int32_t K, int64_t ldx, int64_t ldw, int64_t ldo, const float* cos_t,
                             const float* sin_t, int32_t seq_len, int32_t rope_heads);

/* ---- Gated MLP activation: GatedMLP.forward, src/olmax/nn/mlp.py:69-73:
 * out = act(gate) * up, act 0 = silu, 1 = tanh-approximated gelu (jax.nn.gelu default,
 * src/olmax/nn/transformer/layer.py:133). */
int32_t olmax_glu_fwd(olmax_stream_t stream, const void* gate, const void* up, void* out, int64_t T,
                      int32_t F, int64_t ldg, int64_t ldu, int64_t ldo, int32_t act);
int32_t olmax_glu_bwd(olmax_stream_t stream, const void* gate, const void* up, const void* dh,
                      void* dgate, void* dup, int64_t T, int32_t F, int64_t ldg, int64_t ldu,
                      int64_t lddh, int64_t lddg, int64_t lddu, int32_t act);

/* ---- Attention: AttentionKernel.forward, src/olmax/nn/attention.py:52-109
 * (jax.nn.dot_product_attention(is_causal=True, local_window_size=window)).
 * BSHD: q [B*S, ldq] with head h at columns h*D.., k/v with KH heads (GQA: query head h reads
 * kv head h / (H/KH)).  window < 0: global; window >= 0: keys i-window..i.  softcap > 0:
 * scores <- softcap*tanh(scores/softcap) (extension, not in the reference).
 * lse: fp32 [B, H, S], saved for the backward. */
int32_t olmax_attn_fwd(olmax_stream_t stream, const void* q, const void* k, const void* v, void* o,
                       float* lse, int32_t B, int32_t S, int32_t H, int32_t KH, int32_t D, int64_t ldq,
                       int64_t ldk, int64_t ldv, int64_t ldo, int32_t window, float softcap);
int64_t olmax_attn_bwd_workspace_bytes(int32_t B, int32_t S, int32_t H, int32_t KH, int32_t D);
/* The part of that size the MFMA path needs (delta, [B, H, S] fp32): enough when head_dim is 128
 * and every operand is 16-byte aligned with row strides that are multiples of 8. */
int64_t olmax_attn_bwd_workspace_bytes_aligned(int32_t B, int32_t S, int32_t H);
int32_t olmax_attn_bwd(olmax_stream_t stream, const void* q, const void* k, const void* v,
                       const void* o, const float* lse, const void* d_o, void* dq, void* dk, void* dv,
                       void* workspace, int64_t workspace_bytes, int32_t B, int32_t S, int32_t H,
                       int32_t KH, int32_t D, int64_t ldq, int64_t ldk, int64_t ldv, int64_t ldo,
                       int64_t lddo, int64_t lddq, int64_t lddk, int64_t lddv, int32_t window,
                       float softcap);

/* olmax_attn_bwd without a workspace argument.  No counterpart in the reference: it exists for
 * callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  The delta scratch ([B, H, S] fp32) lives in a device array
 * inside the library (4 MiB per GPU, held until the process ends): batch*heads*seq_len must not
 * exceed olmax_attn_bwd_noalloc_max_rows() (2^20), head_dim must be 128 and every pointer 16-byte
 * aligned with row strides that are multiples of 8, otherwise an error is returned and nothing
 * is launched.  Calls no hipMalloc / hipFree.  All calls on one GPU share the array: calls that
 * overlap on one GPU (different streams or threads) race.  Results equal olmax_attn_bwd's bit for
 * bit (same kernels).
 * Set-up: the scratch address is resolved per device by olmax_attn_bwd_noalloc_init() (device
 * current; no stream work, no allocation) or, failing that, by the first eager call.  Before the
 * entry point is recorded into a HIP graph one of the two must have happened on that device: a
 * first use under stream capture returns an error instead of querying the symbol there. */
int32_t olmax_attn_bwd_noalloc_init(void);
int64_t olmax_attn_bwd_noalloc_max_rows(void);
int32_t olmax_attn_bwd_noalloc(olmax_stream_t stream, const void* q, const void* k, const void* v,
                               const void* o, const float* lse, const void* d_o, void* dq, void* dk,
                               void* dv, int32_t B, int32_t S, int32_t H, int32_t KH, int32_t D,
                               int64_t ldq, int64_t ldk, int64_t ldv, int64_t ldo, int64_t lddo,
                               int64_t lddq, int64_t lddk, int64_t lddv, int32_t window, float softcap);

/* ---- Cross entropy: cross_entropy_loss / fused_cross_entropy_loss,
 * src/olmax/nn/functional.py:70-121 (reduction "mean"; see the label quirks there).
 * logits bf16 (logits_f32 == 0) or fp32; dlogits (optional, may alias logits) receives
 * dloss * d loss / d logits; lse_out (optional [T]) the log-normaliser * (label != ignore). */
int64_t olmax_cross_entropy_workspace_bytes(int64_t T);
int32_t olmax_cross_entropy(olmax_stream_t stream, const void* logits, void* dlogits,
                            const int32_t* labels, float* loss, float* lse_out, void* workspace,
                            int64_t workspace_bytes, int64_t T, int32_t V, int64_t ld, int64_t ldd,
                            int32_t logits_f32, int32_t ignore_index, float softcap, float dloss);
/* The same with the reference's other reductions (src/olmax/nn/functional.py:84-91): reduction 0
 * "mean", 1 "sum", 2 "none".  With "none" `loss` is the [T] array of row losses (0 for ignored and
 * out-of-range labels) and the cotangent of row t is dloss * dloss_rows[t] (dloss_rows: device
 * fp32 [T], NULL = ones). */
int32_t olmax_cross_entropy_reduce(olmax_stream_t stream, const void* logits, void* dlogits,
                                   const int32_t* labels, float* loss, float* lse_out,
                                   const float* dloss_rows, void* workspace, int64_t workspace_bytes,
                                   int64_t T, int32_t V, int64_t ld, int64_t ldd, int32_t logits_f32,
                                   int32_t ignore_index, float softcap, float dloss, int32_t reduction);

/* ---- LM head + cross entropy, forward and backward in one call (three GEMMs around a row kernel;
 * the bf16 logits [T, V] are materialised once in the workspace and overwritten by their gradient,
 * never as fp32 and never twice): LMHead.forward,
 * src/olmax/nn/lm_head.py:59-61, followed by cross_entropy_loss as in the benchmark's
 * loss_fun, src/integration_tests/train_transformer.py:190-206.
 * dh / dW may be NULL to skip.  dw_f32 != 0: dW is fp32. */
int64_t olmax_lmhead_ce_workspace_bytes(int64_t T, int32_t V);
int32_t olmax_lmhead_ce(olmax_stream_t stream, const void* h, const void* W, const int32_t* labels,
                        float* loss, void* dh, void* dW, void* workspace, int64_t workspace_bytes,
                        int64_t T, int32_t d, int32_t V, int32_t ignore_index, float softcap,
                        int32_t dw_f32);

/* ---- Synthetic token batches: _randomize_start_offsets, src/olmax/data/utils.py:12-33:
 * inputs[b, s] = (s + start_offsets[b]) mod V, targets = inputs + 1 (so a target equals V when
 * the input is V - 1).  start_offsets: [B] int32 in [0, V-1), device memory, drawn by the caller. */
int32_t olmax_sequential_tokens(olmax_stream_t stream, const int32_t* start_offsets, int32_t* inputs,
                                int32_t* targets, int32_t B, int32_t S, int32_t V);

/* ---- Embedding: Embedding.forward, src/olmax/nn/embedding.py:30-32 (row gather) and its
 * transpose (scatter-add; dW fp32 is ACCUMULATED into). */
int32_t olmax_embed_fwd(olmax_stream_t stream, const int32_t* ids, const void* W, void* out, int64_t T,
                        int32_t d, int32_t V);
int32_t olmax_embed_bwd(olmax_stream_t stream, const int32_t* ids, const void* dh, float* dW, int64_t T,
                        int32_t d, int32_t V);

/* ---- AdamW: optax.adamw as built by AdamWConfig.build, src/olmax/optim/config.py:136-156,
 * applied with eqx.apply_updates at src/olmax/train/trainer.py:745-752.  In place on fp32
 * p/m/v; g bf16 or fp32 (scaled by grad_scale first: global-norm clipping,
 * src/olmax/optim/utils.py:22-38); `step` is the 1-based count; shadow_bf16 (optional)
 * receives bf16(p_new), replacing cast_tree(params, bf16) of trainer.py:728. */
int32_t olmax_adamw(olmax_stream_t stream, float* p, const void* g, float* m, float* v,
                    void* shadow_bf16, int64_t n, int32_t grad_is_bf16, float lr, float b1, float b2,
                    float eps, float wd, int64_t step, float grad_scale);
/* As olmax_adamw with an extra device-resident multiplier of the gradient (NULL = none). */
int32_t olmax_adamw_dscale(olmax_stream_t stream, float* p, const void* g, float* m, float* v,
                           void* shadow_bf16, int64_t n, int32_t grad_is_bf16, float lr, float b1,
                           float b2, float eps, float wd, int64_t step, float grad_scale,
                           const float* grad_scale_dev);
/* As olmax_adamw_dscale with the step-dependent scalars in device memory: hyper_dev = fp32
 * {lr, 1 - b1^step, 1 - b2^step}, written by earlier work on the same stream.  For hosts whose
 * schedule and step count are device values (optax's inject_hyperparams state inside a jitted
 * step, src/olmax/optim/config.py:141-148): no host read-back, no recompilation per step. */
int32_t olmax_adamw_dev(olmax_stream_t stream, float* p, const void* g, float* m, float* v, void* shadow_bf16,
                        int64_t n, int32_t grad_is_bf16, float b1, float b2, float eps, float wd,
                        const float* hyper_dev, const float* grad_scale_dev);
/* *out += sum(g^2): building block of get_global_norm, src/olmax/jax_utils.py:88-102. */
int32_t olmax_sumsq(olmax_stream_t stream, const void* g, int64_t n, int32_t is_bf16, float* out);

/* ---- utilities */
int32_t olmax_cast_f32_to_bf16(olmax_stream_t stream, const float* in, void* out, int64_t n);
int32_t olmax_cast_bf16_to_f32(olmax_stream_t stream, const void* in, float* out, int64_t n);
int32_t olmax_fill_zero(olmax_stream_t stream, void* p, int64_t nbytes);
int32_t olmax_add_bf16(olmax_stream_t stream, const void* a, const void* b, void* out, int64_t n);

/* =====================================================================================
 * Whole block / whole model: the granularity Transformer.forward
 * (src/olmax/nn/transformer/model.py:95-136) and process_microbatch
 * (src/olmax/train/trainer.py:759-777) run at.
 * ===================================================================================== */
typedef struct {
  int32_t vocab, d_model, n_layers, n_heads, n_kv_heads, head_dim, hidden;
  int32_t layer_type; /* 0 TransformerLayer (pre-norm, layer.py:80-94), 1 ReorderedNorm
                         (layer.py:102-116), 2 Gemma pre+post (layer.py:169-185) */
  int32_t act;        /* 0 silu, 1 gelu-tanh */
  int32_t qk_norm;    /* 0 off; 1 head-wise QK-norm, weight [head_dim] shared by the heads
                         (attention.py:293-296); 2 full width, weights [n_heads*head_dim] for q and
                         [n_kv_heads*head_dim] for k, before the reshape (attention.py:281-284) */
  int32_t tied;       /* LM head shares the embedding matrix (extension) */
  int32_t batch, seq_len;
  int32_t checkpoint; /* 1: full-block activation checkpointing (NothingSaveable,
                         src/olmax/activation_checkpointing.py:71-80); 0: keep activations */
  float eps, attn_softcap, final_softcap;
} olmax_model_config;

/* One parameter leaf inside the flat parameter buffer. */
typedef struct {
  int32_t kind;   /* OLMAX_LEAF_* */
  int32_t layer;  /* -1 for global leaves */
  int64_t offset; /* element offset in the flat fp32 master / bf16 working / bf16 grad buffers */
  int64_t numel;
  int32_t rows, cols;
  int32_t grad_f32;     /* 1: gradient lives in the fp32 grad buffer at grad_f32_offset */
  int64_t grad_f32_offset;
} olmax_leaf;

enum {
  OLMAX_LEAF_EMBEDDING = 0, OLMAX_LEAF_Q, OLMAX_LEAF_K, OLMAX_LEAF_V, OLMAX_LEAF_O,
  OLMAX_LEAF_GATE, OLMAX_LEAF_UP, OLMAX_LEAF_DOWN, OLMAX_LEAF_ATTN_NORM, OLMAX_LEAF_MLP_NORM,
  OLMAX_LEAF_ATTN_IN_NORM, OLMAX_LEAF_MLP_IN_NORM, OLMAX_LEAF_Q_NORM, OLMAX_LEAF_K_NORM,
  OLMAX_LEAF_FINAL_NORM, OLMAX_LEAF_LM_HEAD
};

/* Host-only layout queries. */
int64_t olmax_model_num_params(const olmax_model_config* cfg);
int64_t olmax_model_grad_f32_elems(const olmax_model_config* cfg);
int32_t olmax_model_layout(const olmax_model_config* cfg, olmax_leaf* out, int32_t max_leaves);
int64_t olmax_model_workspace_bytes(const olmax_model_config* cfg);

/* loss + all gradients of one micro-batch: compute_loss_and_grads,
 * src/olmax/train/trainer.py:723-740.
 * params_bf16: flat bf16 working copy; ids/labels int32 [batch*seq_len];
 * windows: host array [n_layers] (-1 = global); cos/sin: host arrays of n_layers device
 * pointers to fp32 [seq_len, head_dim/2] tables (per-layer RoPE theta);
 * grad_bf16 (flat, same offsets as params) and grad_f32 receive the gradients; loss: device
 * fp32 scalar. */
int32_t olmax_model_loss_and_grads(olmax_stream_t stream, const olmax_model_config* cfg,
                                   const int32_t* windows, const float* const* cos_tables,
                                   const float* const* sin_tables, const void* params_bf16,
                                   const int32_t* ids, const int32_t* labels, float* loss,
                                   void* grad_bf16, float* grad_f32, void* workspace,
                                   int64_t workspace_bytes);
/* Forward only (loss). */
int32_t olmax_model_loss(olmax_stream_t stream, const olmax_model_config* cfg, const int32_t* windows,
                         const float* const* cos_tables, const float* const* sin_tables,
                         const void* params_bf16, const int32_t* ids, const int32_t* labels,
                         float* loss, void* workspace, int64_t workspace_bytes);

/* step_optimizer, src/olmax/train/trainer.py:742-757: fused AdamW over every leaf.
 * leaf_decay: host array with one entry per leaf in olmax_model_layout order, 0 = the leaf is
 * exempt from weight decay, the mask of OptimConfig.build_weight_decay_mask
 * (src/olmax/optim/config.py:94-122; the benchmark exempts "embedding.weight",
 * src/integration_tests/train_transformer.py:388); NULL = every leaf decays.  max_grad_norm > 0 applies
 * clip_grads_by_global_norm (src/olmax/optim/utils.py:22-38); norm_scratch: device float[2], left holding
 * {clip factor, gradient norm}.  hyper_dev (optional, as in olmax_adamw_dev): device fp32
 * {lr, 1 - b1^step, 1 - b2^step}; when given, the host `step` and `lr` arguments are ignored. */
int32_t olmax_model_adamw(olmax_stream_t stream, const olmax_model_config* cfg, float* master,
                          float* m, float* v, void* params_bf16, const void* grad_bf16,
                          const float* grad_f32, int64_t step, float lr, float b1, float b2, float eps,
                          float wd, const int32_t* leaf_decay, float max_grad_norm, float* norm_scratch,
                          const float* hyper_dev);

/* Gradient accumulation over micro-batches: optax.MultiSteps as built at
 * src/olmax/optim/config.py:153-154 and driven once per micro-batch by train_batch,
 * src/olmax/train/trainer.py:779-807.  acc: fp32 [olmax_model_num_params], parameter layout;
 * micro-batch mini_step (0-based) enters the running mean acc += (g - acc) / (mini_step + 1)
 * (mini_step 0 overwrites).  olmax_grad_accumulate is the same for one flat array. */
int32_t olmax_grad_accumulate(olmax_stream_t stream, float* acc, const void* g, int64_t n, int32_t grad_is_bf16,
                              int32_t mini_step);
int32_t olmax_model_grad_accumulate(olmax_stream_t stream, const olmax_model_config* cfg, float* acc,
                                    const void* grad_bf16, const float* grad_f32, int32_t mini_step);
/* AdamW (+ optional global-norm clip of the accumulated mean) from acc: the update MultiSteps
 * applies on the last micro-batch of a batch. */
int32_t olmax_model_adamw_accumulated(olmax_stream_t stream, const olmax_model_config* cfg, float* master,
                                      float* m, float* v, void* params_bf16, const float* acc, int64_t step,
                                      float lr, float b1, float b2, float eps, float wd,
                                      const int32_t* leaf_decay, float max_grad_norm, float* norm_scratch,
                                      const float* hyper_dev);

/* process_microbatch, src/olmax/train/trainer.py:759-777: loss + gradients + AdamW in one call.
 * opt_stream (optional, default priority, != stream): when given, clipping is off and the config
 * checkpoints its blocks, each layer's AdamW runs there concurrently with the recompute and
 * backward of the layers below it, and `stream` waits for it at the end; otherwise AdamW follows
 * the backward pass on `stream`.  Creates one HIP event per host thread on first use. */
int32_t olmax_model_train_step(olmax_stream_t stream, olmax_stream_t opt_stream, const olmax_model_config* cfg,
                               const int32_t* windows, const float* const* cos_tables,
                               const float* const* sin_tables, float* master, float* m, float* v,
                               void* params_bf16, const int32_t* ids, const int32_t* labels, float* loss,
                               void* grad_bf16, float* grad_f32, void* workspace, int64_t workspace_bytes,
                               int64_t step, float lr, float b1, float b2, float eps, float wd,
                               const int32_t* leaf_decay, float max_grad_norm, float* norm_scratch,
                               const float* hyper_dev);

/* Single transformer block in isolation (any of the three orderings). */
typedef struct {
  const void *wqkv, *wo, *wgu, *wdown;          /* bf16: [(H+2K)D, d], [d, HD], [2F, d], [d, F] */
  const void *attn_norm, *mlp_norm;             /* bf16 [d] */
  const void *attn_in_norm, *mlp_in_norm;       /* bf16 [d], Gemma only */
  const void *q_norm, *k_norm;                  /* bf16 [D], qk_norm only */
} olmax_block_weights;
typedef struct {
  void *wqkv, *wo, *wgu, *wdown;                /* bf16, overwritten */
  float *attn_norm, *mlp_norm, *attn_in_norm, *mlp_in_norm, *q_norm, *k_norm; /* fp32, accumulated */
} olmax_block_grads;
int64_t olmax_block_acts_bytes(const olmax_model_config* cfg);
int64_t olmax_block_tmp_bytes(const olmax_model_config* cfg);
int32_t olmax_block_fwd(olmax_stream_t stream, const olmax_model_config* cfg, const olmax_block_weights* w,
                        int32_t window, const float* cos_t, const float* sin_t, const void* x, void* y,
                        void* acts, int64_t acts_bytes);
int32_t olmax_block_bwd(olmax_stream_t stream, const olmax_model_config* cfg, const olmax_block_weights* w,
                        const olmax_block_grads* g, int32_t window, const float* cos_t,
                        const float* sin_t, const void* x, const void* dy, void* dx, void* acts,
                        int64_t acts_bytes, void* tmp, int64_t tmp_bytes);

/* =====================================================================================
 * Diagnostics.  Process-wide switches (atomics): they change what EVERY thread's later calls do,
 * are meant for tests, tuning and profiling runs, and are not for use while other threads are
 * inside the library or under graph capture.
 * ===================================================================================== */
/* Force the MFMA tile variant of olmax_gemm_bf16 (0 = automatic, 128, 256).  While set, the
 * fused GLU / RoPE projections take their unfused paths (same results). */
void olmax_gemm_set_tile(int tile);
/* Order in which the MFMA GEMM's workgroups take their tiles: 0 = automatic (per shape and operand
 * layout), -1 = one contiguous run of tiles per XCD, n > 0 = windows of 8 x 4 tiles per XCD whose 8
 * windows in flight cover n strips of 8 tile rows (n = 1, 2, 4, 8).  Results do not depend on it. */
void olmax_gemm_set_order(int order);
/* Record a HIP-event pair on the launch stream around every MFMA GEMM launch between begin and
 * end (allocates events).  end() waits for them and aggregates per kernel instantiation:
 * key = tile | a_kc<<12 | b_kc<<13 | has_res<<14 | out_f32<<15 | glu_epilogue<<16 |
 * rope_epilogue<<17; ms = summed durations, flops / bytes = summed algorithmic work (2MNK;
 * operands and result moved once).  Returns the number of distinct keys written (at most cap). */
void olmax_gemm_profile_begin(void);
int32_t olmax_gemm_profile_end(int32_t* keys, double* ms, double* flops, double* bytes, int64_t* launches,
                               int32_t cap);
/* The same, aggregated per (key, M, N, K): mnk receives three ints per entry. */
int32_t olmax_gemm_profile_end_shapes(int32_t* keys, int32_t* mnk, double* ms, int64_t* launches, int32_t cap);
/* Profiler ranges: the counterpart of the reference's jax.named_scope annotations and
 * ProfilerCallback (src/olmax/train/callbacks/profiler.py:33-50).  on != 0: the whole-model entry
 * points emit roctx ranges ("olmax.layers.<l>.forward" / ".backward", "olmax.lm_head_and_loss")
 * on the calling host thread, visible to rocprofv3 --marker-trace.  Needs a roctx library at run
 * time; returns an error (and stays off) without it. */
int32_t olmax_set_profiler_ranges(int32_t on);
/* Number of AdamW launch groups the calling thread's last olmax_model_train_step put on its
 * optimizer stream; 0 means that step ran AdamW after the backward pass on the main stream
 * (no second stream, clipping on, or activations kept).  For tests of the overlapped path. */
int32_t olmax_model_last_step_overlapped_launches(void);

#ifdef __cplusplus
}
#endif
#endif /* OLMAX_HIP_H */
