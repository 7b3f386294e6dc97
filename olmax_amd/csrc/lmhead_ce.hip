// Cross-entropy over the full vocabulary and the fused LM-head + CE forward/backward.
//
// Reference semantics: cross_entropy_loss, src/olmax/nn/functional.py:70-91 (reduction
// "mean" over labels != ignore_index; an out-of-range label contributes zero loss and zero
// gradient but still counts in the denominator), fed by LMHead.forward,
// src/olmax/nn/lm_head.py:59-61 (logits = bf16 GEMM output widened to fp32).
//
// One block owns one row of logits.  bf16 rows of up to 163840 entries are loaded ONCE into the
// block's registers (128-bit loads), reduced to max and sum-exp, and written back as
// d logits = (softmax - onehot) * dloss / n_counted from the registers; longer or fp32 rows take
// the streaming form (online max / sum-exp in pass 1, a second read of the row in pass 2).
// Optional final-logit soft-cap z = c*tanh(x/c) is applied on the fly in both passes.
#include "common.h"

extern "C" int32_t olmax_gemm_bf16(hipStream_t stream, const void* A, const void* B, void* C,
                                   const void* R, int32_t M, int32_t N, int32_t K, int64_t lda,
                                   int64_t ldb, int64_t ldc, int64_t ldr, int32_t a_layout,
                                   int32_t b_layout, int32_t out_f32);

namespace {

__global__ __launch_bounds__(256) void ce_count_kernel(const int32_t* __restrict__ labels, int64_t T,
                                                       int32_t ignore_index, int32_t* __restrict__ n_out) {
  __shared__ float red[4];
  float c = 0.f;
  for (int64_t i = threadIdx.x; i < T; i += 256) c += labels[i] != ignore_index ? 1.f : 0.f;
  c = block_sum<4>(c, red);
  if (threadIdx.x == 0) *n_out = (int32_t)(c + 0.5f);
}

template <typename T> struct Io;
template <> struct Io<bf16> {
  static constexpr int VEC = 8;
  static __device__ __forceinline__ void load(const bf16* p, float* f) {
    Pack8 t;
    t.u = *reinterpret_cast<const u32x4*>(p);
#pragma unroll
    for (int e = 0; e < 8; e++) f[e] = bf2f(t.e[e]);
  }
  static __device__ __forceinline__ void store(bf16* p, const float* f) {
    Pack8 t;
#pragma unroll
    for (int e = 0; e < 8; e++) t.e[e] = f2bf(f[e]);
    *reinterpret_cast<u32x4*>(p) = t.u;
  }
  static __device__ __forceinline__ float ld1(const bf16* p) { return bf2f(*p); }
  static __device__ __forceinline__ void st1(bf16* p, float f) { *p = f2bf(f); }
};
template <> struct Io<float> {
  static constexpr int VEC = 4;
  static __device__ __forceinline__ void load(const float* p, float* f) {
    f32x4 t = *reinterpret_cast<const f32x4*>(p);
#pragma unroll
    for (int e = 0; e < 4; e++) f[e] = t[e];
  }
  static __device__ __forceinline__ void store(float* p, const float* f) {
    f32x4 t;
#pragma unroll
    for (int e = 0; e < 4; e++) t[e] = f[e];
    *reinterpret_cast<f32x4*>(p) = t;
  }
  static __device__ __forceinline__ float ld1(const float* p) { return *p; }
  static __device__ __forceinline__ void st1(float* p, float f) { *p = f; }
};

template <typename T, bool CAP>
__global__ __launch_bounds__(256) void ce_row_kernel(
    const T* __restrict__ logits, T* __restrict__ dlogits, const int32_t* __restrict__ labels,
    float* __restrict__ row_loss, float* __restrict__ lse_out, const int32_t* __restrict__ n_counted,
    int64_t rows, int V, int64_t ld, int64_t ldd, int32_t ignore_index, float cap, float dloss,
    int vec_ok, const float* __restrict__ drow, int mean) {
  constexpr int VEC = Io<T>::VEC;
  __shared__ float red[4];
  __shared__ float label_logit;
  const int64_t row = blockIdx.x;
  const T* zr = logits + row * ld;
  const int label = labels[row];
  const float inv_cap = CAP ? 1.f / cap : 0.f;
  const bool counted = label != ignore_index;
  const bool inrange = label >= 0 && label < V;
  // The label's logit is fetched and parked in LDS BEFORE the first block barrier: with dlogits
  // aliasing logits, other waves overwrite the row as soon as they are past the last reduction,
  // and no load of the row may be left to race with those stores.
  if (threadIdx.x == 0) {
    float zl = 0.f;
    if (counted && inrange) {
      zl = Io<T>::ld1(zr + label);
      if (CAP) zl = cap * fast_tanh(zl * inv_cap);
    }
    label_logit = zl;
  }
  // ---- pass 1: online max / sum-exp ----
  float mx = -INFINITY, sm = 0.f;
  const int nvec = vec_ok ? V / VEC : 0;
  for (int i = threadIdx.x; i < nvec; i += 256) {
    float f[VEC];
    Io<T>::load(zr + i * VEC, f);
    float cm = -INFINITY;
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      if (CAP) f[e] = cap * fast_tanh(f[e] * inv_cap);
      cm = fmaxf(cm, f[e]);
    }
    if (cm > mx) {
      sm *= __expf(mx - cm);
      mx = cm;
    }
#pragma unroll
    for (int e = 0; e < VEC; e++) sm += __expf(f[e] - mx);
  }
  for (int i = nvec * VEC + threadIdx.x; i < V; i += 256) {
    float f = Io<T>::ld1(zr + i);
    if (CAP) f = cap * fast_tanh(f * inv_cap);
    if (f > mx) {
      sm *= __expf(mx - f);
      mx = f;
    }
    sm += __expf(f - mx);
  }
  const float gmx = block_max<4>(mx, red);
  sm = (mx == -INFINITY) ? 0.f : sm * __expf(mx - gmx);
  const float gsm = block_sum<4>(sm, red);
  const float lse = gmx + __logf(gsm);
  if (threadIdx.x == 0) {
    row_loss[row] = (counted && inrange) ? (lse - label_logit) : 0.f;
    if (lse_out) lse_out[row] = counted ? lse : 0.f;
  }
  if (!dlogits) return;
  // ---- pass 2: gradient, in place allowed ----
  T* dr = dlogits + row * ldd;
  // d(reduced loss) / d(row loss): 1/n for "mean", 1 for "sum", the row's own cotangent for "none"
  const float scale = (counted && inrange) ? dloss * (drow ? drow[row] : 1.f) / (mean ? (float)(*n_counted) : 1.f) : 0.f;
  for (int i = threadIdx.x; i < nvec; i += 256) {
    float f[VEC];
    Io<T>::load(zr + i * VEC, f);
#pragma unroll
    for (int e = 0; e < VEC; e++) {
      float z = f[e], chain = 1.f;
      if (CAP) {
        const float t = fast_tanh(z * inv_cap);
        z = cap * t;
        chain = 1.f - t * t;
      }
      float p = __expf(z - lse);
      if (i * VEC + e == label) p -= 1.f;
      f[e] = p * scale * chain;
    }
    Io<T>::store(dr + i * VEC, f);
  }
  for (int i = nvec * VEC + threadIdx.x; i < V; i += 256) {
    float z = Io<T>::ld1(zr + i), chain = 1.f;
    if (CAP) {
      const float t = fast_tanh(z * inv_cap);
      z = cap * t;
      chain = 1.f - t * t;
    }
    float p = __expf(z - lse);
    if (i == label) p -= 1.f;
    Io<T>::st1(dr + i, p * scale * chain);
  }
}

// The same row computation for bf16 rows short enough to keep in registers between the two
// passes (THREADS x MAXV vectors of 8): the logits are read from memory once and the gradient
// written once, 4 B per logit instead of 6.  Max and sum-exp are two plain block reductions (no
// online rescaling needed when the whole row is at hand).
template <bool CAP, int THREADS, int MAXV>
__global__ __launch_bounds__(THREADS) void ce_row_regs_kernel(
    const bf16* __restrict__ logits, bf16* __restrict__ dlogits, const int32_t* __restrict__ labels,
    float* __restrict__ row_loss, float* __restrict__ lse_out, const int32_t* __restrict__ n_counted,
    int V, int64_t ld, int64_t ldd, int32_t ignore_index, float cap, float dloss,
    const float* __restrict__ drow, int mean) {
  constexpr int NW = THREADS / 64;
  __shared__ float red[NW];
  __shared__ float label_logit;
  const int64_t row = blockIdx.x;
  const bf16* zr = logits + row * ld;
  const int label = labels[row];
  const float inv_cap = CAP ? 1.f / cap : 0.f;
  const int nvec = V / 8;
  const bool counted = label != ignore_index;
  const bool inrange = label >= 0 && label < V;
  // label logit into LDS before the first barrier (see ce_row_kernel): nothing reads the row
  // from memory once any wave may be storing the gradient over it
  if (threadIdx.x == 0) {
    float zl = 0.f;
    if (counted && inrange) {
      zl = bf2f(zr[label]);
      if (CAP) zl = cap * fast_tanh(zl * inv_cap);
    }
    label_logit = zl;
  }
  Pack8 c[MAXV];
#pragma unroll
  for (int i = 0; i < MAXV; i++) {
    const int idx = i * THREADS + threadIdx.x;
    if (idx < nvec) c[i].u = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(zr) + idx);
  }
  auto value = [&](bf16 x) {
    const float f = bf2f(x);
    return CAP ? cap * fast_tanh(f * inv_cap) : f;
  };
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < MAXV; i++)
    if (i * THREADS + threadIdx.x < nvec) {
#pragma unroll
      for (int e = 0; e < 8; e++) mx = fmaxf(mx, value(c[i].e[e]));
    }
  const float gmx = block_max<NW>(mx, red);
  float sm = 0.f;
#pragma unroll
  for (int i = 0; i < MAXV; i++)
    if (i * THREADS + threadIdx.x < nvec) {
#pragma unroll
      for (int e = 0; e < 8; e++) sm += __expf(value(c[i].e[e]) - gmx);
    }
  const float gsm = block_sum<NW>(sm, red);
  const float lse = gmx + __logf(gsm);
  if (threadIdx.x == 0) {
    row_loss[row] = (counted && inrange) ? (lse - label_logit) : 0.f;
    if (lse_out) lse_out[row] = counted ? lse : 0.f;
  }
  if (!dlogits) return;
  bf16* dr = dlogits + row * ldd;
  // d(reduced loss) / d(row loss): 1/n for "mean", 1 for "sum", the row's own cotangent for "none"
  const float scale = (counted && inrange) ? dloss * (drow ? drow[row] : 1.f) / (mean ? (float)(*n_counted) : 1.f) : 0.f;
#pragma unroll
  for (int i = 0; i < MAXV; i++) {
    const int idx = i * THREADS + threadIdx.x;
    if (idx < nvec) {
      Pack8 o;
#pragma unroll
      for (int e = 0; e < 8; e++) {
        float z = bf2f(c[i].e[e]), chain = 1.f;
        if (CAP) {
          const float t = fast_tanh(z * inv_cap);
          z = cap * t;
          chain = 1.f - t * t;
        }
        float p = __expf(z - lse);
        if (idx * 8 + e == label) p -= 1.f;
        o.e[e] = f2bf(p * scale * chain);
      }
      *(reinterpret_cast<u32x4*>(dr) + idx) = o.u;
    }
  }
}

// loss = sum(row_loss) / n_counted, or the plain sum (single block; deterministic order)
__global__ __launch_bounds__(256) void ce_finalize_kernel(const float* __restrict__ row_loss, int64_t T,
                                                          const int32_t* __restrict__ n_counted,
                                                          float* __restrict__ loss, int mean) {
  __shared__ float red[4];
  float s = 0.f;
  for (int64_t i = threadIdx.x; i < T; i += 256) s += row_loss[i];
  s = block_sum<4>(s, red);
  if (threadIdx.x == 0) *loss = mean ? s / (float)(*n_counted) : s;
}

}  // namespace

// Workspace: T floats (row losses) + 16 bytes (counted-row count), 16-byte aligned.
extern "C" int64_t olmax_cross_entropy_workspace_bytes(int64_t T) { return ((T * 4 + 15) / 16) * 16 + 16; }

// logits [T, V] (bf16 when logits_f32 == 0, else fp32) -> loss (device fp32: a scalar, or [T] row
// losses for reduction "none"); dlogits (same dtype, may alias logits, may be NULL) <-
// d loss / d logits times the incoming cotangent (the scalar dloss; for "none" also the per-row
// device array dloss_rows when given); lse_out (optional, [T]) <- log-normaliser *
// (label != ignore_index)  (the reference's fused_cross_entropy_loss second output,
// src/olmax/nn/functional.py:94-121).  reduction: 0 "mean", 1 "sum", 2 "none" (functional.py:84-91).
extern "C" int32_t olmax_cross_entropy_reduce(hipStream_t stream, const void* logits, void* dlogits,
                                              const int32_t* labels, float* loss, float* lse_out,
                                              const float* dloss_rows, void* workspace, int64_t workspace_bytes,
                                              int64_t T, int32_t V, int64_t ld, int64_t ldd, int32_t logits_f32,
                                              int32_t ignore_index, float softcap, float dloss, int32_t reduction) {
  OLMAX_CHECK(logits && labels && loss && workspace, OLMAX_ERR_ARG, "olmax_cross_entropy: null pointer");
  OLMAX_CHECK(T > 0 && V > 0 && ld >= V && (!dlogits || ldd >= V), OLMAX_ERR_SHAPE, "olmax_cross_entropy: bad shape T=%ld V=%d", (long)T, V);
  OLMAX_CHECK(reduction >= 0 && reduction <= 2, OLMAX_ERR_ARG, "olmax_cross_entropy: reduction must be 0 (mean), 1 (sum) or 2 (none)");
  OLMAX_CHECK(!dloss_rows || reduction == 2, OLMAX_ERR_ARG, "olmax_cross_entropy: a per-row cotangent only goes with reduction none");
  OLMAX_CHECK(workspace_bytes >= olmax_cross_entropy_workspace_bytes(T) && aligned16(workspace), OLMAX_ERR_WORKSPACE, "olmax_cross_entropy: workspace too small or misaligned");
  // "none": the row kernels write the row losses straight into the caller's array
  float* row_loss = reduction == 2 ? loss : (float*)workspace;
  int32_t* n_counted = (int32_t*)((char*)workspace + ((T * 4 + 15) / 16) * 16);
  const int mean = reduction == 0;
  hipLaunchKernelGGL(ce_count_kernel, dim3(1), dim3(256), 0, stream, labels, T, ignore_index, n_counted);
  const int vecw = logits_f32 ? 4 : 8;
  const int vec_ok = aligned16(logits) && (!dlogits || aligned16(dlogits)) && ld % vecw == 0 && (!dlogits || ldd % vecw == 0);
  const bool cap = softcap > 0.f;
  dim3 grid((unsigned)T);
#define CE_GO(TY, CAPV)                                                                          \
  hipLaunchKernelGGL((ce_row_kernel<TY, CAPV>), grid, dim3(256), 0, stream, (const TY*)logits,   \
                     (TY*)dlogits, labels, row_loss, lse_out, n_counted, T, V, ld, ldd,          \
                     ignore_index, softcap, dloss, vec_ok, dloss_rows, mean)
#define CE_REGS(CAPV, TH, MV)                                                                              \
  hipLaunchKernelGGL((ce_row_regs_kernel<CAPV, TH, MV>), grid, dim3(TH), 0, stream, (const bf16*)logits,   \
                     (bf16*)dlogits, labels, row_loss, lse_out, n_counted, V, ld, ldd, ignore_index, softcap, dloss, dloss_rows, mean)
  const bool regs_ok = !logits_f32 && vec_ok && V % 8 == 0;
  if (logits_f32) {
    if (cap) CE_GO(float, true); else CE_GO(float, false);
  } else if (regs_ok && V <= 512 * 8 * 26) {  // up to 106496 logits: 8 waves holding 26 vectors each
    if (cap) CE_REGS(true, 512, 26); else CE_REGS(false, 512, 26);
  } else if (regs_ok && V <= 1024 * 8 * 20) {  // up to 163840 logits: 16 waves holding 20 vectors each (128 registers per lane)
    if (cap) CE_REGS(true, 1024, 20); else CE_REGS(false, 1024, 20);
  } else {
    if (cap) CE_GO(bf16, true); else CE_GO(bf16, false);
  }
#undef CE_GO
#undef CE_REGS
  if (reduction != 2) hipLaunchKernelGGL(ce_finalize_kernel, dim3(1), dim3(256), 0, stream, row_loss, T, n_counted, loss, mean);
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}

// reduction "mean": what the benchmark's loss_fun and the fused LM head use
extern "C" int32_t olmax_cross_entropy(hipStream_t stream, const void* logits, void* dlogits,
                                       const int32_t* labels, float* loss, float* lse_out,
                                       void* workspace, int64_t workspace_bytes, int64_t T, int32_t V,
                                       int64_t ld, int64_t ldd, int32_t logits_f32,
                                       int32_t ignore_index, float softcap, float dloss) {
  return olmax_cross_entropy_reduce(stream, logits, dlogits, labels, loss, lse_out, nullptr, workspace, workspace_bytes, T, V, ld,
                                    ldd, logits_f32, ignore_index, softcap, dloss, 0);
}

// Workspace for the fused LM head: bf16 logits [T, V] + the CE workspace.
extern "C" int64_t olmax_lmhead_ce_workspace_bytes(int64_t T, int32_t V) {
  return ((T * (int64_t)V * 2 + 255) / 256) * 256 + olmax_cross_entropy_workspace_bytes(T);
}

// Fused LM head + cross entropy, forward and backward in one call:
//   logits = h W^T (bf16) ; loss = CE(softcap(logits), labels) ;
//   dlogits overwrites logits in the workspace ; dh = dlogits W ; dW = dlogits^T h.
// h [T, d] bf16, W [V, d] bf16, labels [T] int32.  dh [T, d] bf16 and dW [V, d] (bf16, or
// fp32 when dw_f32 != 0) may be NULL to skip that product (forward-only when both are NULL).
extern "C" int32_t olmax_lmhead_ce(hipStream_t stream, const void* h, const void* W,
                                   const int32_t* labels, float* loss, void* dh, void* dW,
                                   void* workspace, int64_t workspace_bytes, int64_t T, int32_t d,
                                   int32_t V, int32_t ignore_index, float softcap, int32_t dw_f32) {
  OLMAX_CHECK(h && W && labels && loss && workspace, OLMAX_ERR_ARG, "olmax_lmhead_ce: null pointer");
  OLMAX_CHECK(T > 0 && d > 0 && V > 0 && T < (1LL << 31), OLMAX_ERR_SHAPE, "olmax_lmhead_ce: bad shape");
  OLMAX_CHECK(workspace_bytes >= olmax_lmhead_ce_workspace_bytes(T, V) && (((uintptr_t)workspace) & 255) == 0, OLMAX_ERR_WORKSPACE,
              "olmax_lmhead_ce: workspace needs %ld bytes, 256-byte aligned", (long)olmax_lmhead_ce_workspace_bytes(T, V));
  void* logits = workspace;
  void* ce_ws = (char*)workspace + ((T * (int64_t)V * 2 + 255) / 256) * 256;
  int rc = olmax_gemm_bf16(stream, h, W, logits, nullptr, (int)T, V, d, d, d, V, 0, 0, 0, 0);
  if (rc) return rc;
  const bool need_grad = dh || dW;
  rc = olmax_cross_entropy(stream, logits, need_grad ? logits : nullptr, labels, loss, nullptr, ce_ws,
                           olmax_cross_entropy_workspace_bytes(T), T, V, V, V, 0, ignore_index, softcap, 1.f);
  if (rc) return rc;
  if (dh) {
    rc = olmax_gemm_bf16(stream, logits, W, dh, nullptr, (int)T, d, V, V, d, d, 0, 0, 1, 0);
    if (rc) return rc;
  }
  if (dW) {
    rc = olmax_gemm_bf16(stream, logits, h, dW, nullptr, V, d, (int)T, V, d, d, 0, 1, 1, dw_f32);
    if (rc) return rc;
  }
  return OLMAX_OK;
}
