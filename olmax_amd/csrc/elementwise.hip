// HBM-bound elementwise / gather kernels: gated-MLP activation, embedding gather and
// scatter-add, fused fp32 AdamW (with the bf16 working-copy write), utility fills/casts.
// 128-bit accesses, grid-stride loops.
//
// Reference semantics:
//   GatedMLP      src/olmax/nn/mlp.py:69-73 (act = jax.nn.silu; jax.nn.gelu(tanh) for Gemma,
//                 src/olmax/nn/transformer/layer.py:133)
//   Embedding     src/olmax/nn/embedding.py:30-32
//   AdamW         optax.adamw configured at src/olmax/optim/config.py:136-156, applied at
//                 src/olmax/train/trainer.py:745-752; the bf16 copy replaces the per-step
//                 cast_tree(params, bf16) of src/olmax/train/trainer.py:728
#include "common.h"
#include <atomic>

namespace {

// gate/up are column blocks of one [T, ld] buffer (or separate buffers); out [T, F].
template <bool GELU>
__global__ __launch_bounds__(256) void glu_fwd_kernel(const bf16* __restrict__ gate,
                                                      const bf16* __restrict__ up,
                                                      bf16* __restrict__ out, int64_t T, int F,
                                                      int64_t ldg, int64_t ldu, int64_t ldo) {
  const int cpr = F / 8;
  const int64_t total = T * cpr;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t t = i / cpr;
    const int c = (int)(i % cpr) * 8;
    Pack8 g, u, o;
    g.u = *reinterpret_cast<const u32x4*>(gate + t * ldg + c);
    u.u = *reinterpret_cast<const u32x4*>(up + t * ldu + c);
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const float gf = bf2f(g.e[e]);
      const float a = bf2f(f2bf(GELU ? act_gelu(gf) : act_silu(gf)));  // act output is a bf16 array
      o.e[e] = f2bf(a * bf2f(u.e[e]));
    }
    *reinterpret_cast<u32x4*>(out + t * ldo + c) = o.u;
  }
}

template <bool GELU>
__global__ __launch_bounds__(256) void glu_bwd_kernel(const bf16* __restrict__ gate,
                                                      const bf16* __restrict__ up,
                                                      const bf16* __restrict__ dh,
                                                      bf16* __restrict__ dgate,
                                                      bf16* __restrict__ dup, int64_t T, int F,
                                                      int64_t ldg, int64_t ldu, int64_t lddh,
                                                      int64_t lddg, int64_t lddu) {
  const int cpr = F / 8;
  const int64_t total = T * cpr;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t t = i / cpr;
    const int c = (int)(i % cpr) * 8;
    Pack8 g, u, d, og, ou;
    g.u = *reinterpret_cast<const u32x4*>(gate + t * ldg + c);
    u.u = *reinterpret_cast<const u32x4*>(up + t * ldu + c);
    d.u = *reinterpret_cast<const u32x4*>(dh + t * lddh + c);
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const float gf = bf2f(g.e[e]), uf = bf2f(u.e[e]), df = bf2f(d.e[e]);
      og.e[e] = f2bf(df * uf * (GELU ? act_gelu_grad(gf) : act_silu_grad(gf)));
      ou.e[e] = f2bf(df * (GELU ? act_gelu(gf) : act_silu(gf)));
    }
    *reinterpret_cast<u32x4*>(dgate + t * lddg + c) = og.u;
    *reinterpret_cast<u32x4*>(dup + t * lddu + c) = ou.u;
  }
}

template <bool GELU>
__global__ void glu_fwd_scalar(const bf16* gate, const bf16* up, bf16* out, int64_t T, int F,
                               int64_t ldg, int64_t ldu, int64_t ldo) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= T * F) return;
  const int64_t t = i / F;
  const int c = (int)(i % F);
  const float gf = bf2f(gate[t * ldg + c]);
  const float a = bf2f(f2bf(GELU ? act_gelu(gf) : act_silu(gf)));
  out[t * ldo + c] = f2bf(a * bf2f(up[t * ldu + c]));
}
template <bool GELU>
__global__ void glu_bwd_scalar(const bf16* gate, const bf16* up, const bf16* dh, bf16* dgate,
                               bf16* dup, int64_t T, int F, int64_t ldg, int64_t ldu, int64_t lddh,
                               int64_t lddg, int64_t lddu) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= T * F) return;
  const int64_t t = i / F;
  const int c = (int)(i % F);
  const float gf = bf2f(gate[t * ldg + c]), uf = bf2f(up[t * ldu + c]), df = bf2f(dh[t * lddh + c]);
  dgate[t * lddg + c] = f2bf(df * uf * (GELU ? act_gelu_grad(gf) : act_silu_grad(gf)));
  dup[t * lddu + c] = f2bf(df * (GELU ? act_gelu(gf) : act_silu(gf)));
}

// ------------------------------------------------------------------ gradient accumulation
// Running mean over micro-batches, acc += (g - acc) / (k + 1) for the k-th (0-based) micro-batch
// (optax.MultiSteps with use_grad_mean, which the reference wraps its optimizer in,
// src/olmax/optim/config.py:153-154); k = 0 overwrites acc.
template <bool G_BF16>
__global__ __launch_bounds__(256) void grad_accum_kernel(float* __restrict__ acc, const void* __restrict__ gv, int64_t n,
                                                         float inv, int first) {
  const int64_t n4 = n / 4;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (int64_t)gridDim.x * 256) {
    float g[4];
    if (G_BF16) {
      Pack4 gp;
      gp.u = reinterpret_cast<const u32x2*>(gv)[i];
#pragma unroll
      for (int e = 0; e < 4; e++) g[e] = bf2f(gp.e[e]);
    } else {
      const f32x4 gf = reinterpret_cast<const f32x4*>(gv)[i];
#pragma unroll
      for (int e = 0; e < 4; e++) g[e] = gf[e];
    }
    f32x4 a;
    if (first) {
#pragma unroll
      for (int e = 0; e < 4; e++) a[e] = g[e];
    } else {
      a = reinterpret_cast<const f32x4*>(acc)[i];
#pragma unroll
      for (int e = 0; e < 4; e++) a[e] = a[e] + (g[e] - a[e]) * inv;
    }
    reinterpret_cast<f32x4*>(acc)[i] = a;
  }
  if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
    const int64_t i = n4 * 4 + threadIdx.x;
    const float g = G_BF16 ? bf2f(reinterpret_cast<const bf16*>(gv)[i]) : reinterpret_cast<const float*>(gv)[i];
    acc[i] = first ? g : acc[i] + (g - acc[i]) * inv;
  }
}

// ------------------------------------------------------------------ synthetic token batches
// inputs[b, s] = (s + offset[b]) mod V, targets = inputs + 1 (a target equals V, one past the
// vocabulary, whenever the input is V - 1: the loss treats such a label as an all-zero one-hot).
__global__ __launch_bounds__(256) void sequential_tokens_kernel(const int32_t* __restrict__ offsets,
                                                                int32_t* __restrict__ inputs,
                                                                int32_t* __restrict__ targets, int B, int S, int V) {
  const int64_t total = (int64_t)B * S;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int b = (int)(i / S), sidx = (int)(i % S);
    const int32_t tok = (int32_t)(((int64_t)sidx + offsets[b]) % V);
    inputs[i] = tok;
    targets[i] = tok + 1;
  }
}

// ------------------------------------------------------------------ embedding
// ids follow NumPy/JAX indexing of `weight[ids]` (src/olmax/nn/embedding.py:32): a negative id
// counts from the end, and what is still outside [0, V) is clamped (JAX's gather mode for
// out-of-bounds reads; upstream semantics, the data path never produces such ids).  The
// scatter-add is the transpose of exactly that gather.
__device__ __forceinline__ int wrap_clamp_id(int id, int V) {
  if (id < 0) id += V;
  return id < 0 ? 0 : (id >= V ? V - 1 : id);
}
__global__ __launch_bounds__(256) void embed_fwd_kernel(const int32_t* __restrict__ ids,
                                                        const bf16* __restrict__ W,
                                                        bf16* __restrict__ out, int64_t T, int d,
                                                        int V) {
  const int cpr = d / 8;
  const int64_t total = T * cpr;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t t = i / cpr;
    const int c = (int)(i % cpr) * 8;
    const int id = wrap_clamp_id(ids[t], V);
    *reinterpret_cast<u32x4*>(out + t * d + c) = *reinterpret_cast<const u32x4*>(W + (int64_t)id * d + c);
  }
}
__global__ void embed_fwd_scalar(const int32_t* ids, const bf16* W, bf16* out, int64_t T, int d, int V) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= T * d) return;
  const int id = wrap_clamp_id(ids[i / d], V);
  out[i] = W[(int64_t)id * d + i % d];
}
// dW[ids[t], :] += dh[t, :]   (fp32 accumulate; duplicates sum through atomics)
__global__ __launch_bounds__(256) void embed_bwd_kernel(const int32_t* __restrict__ ids,
                                                        const bf16* __restrict__ dh,
                                                        float* __restrict__ dW, int64_t T, int d,
                                                        int V) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < T * d; i += (int64_t)gridDim.x * 256) {
    const int64_t t = i / d;
    const int c = (int)(i % d);
    const int id = wrap_clamp_id(ids[t], V);
    atomicAdd(&dW[(int64_t)id * d + c], bf2f(dh[i]));
  }
}

// ------------------------------------------------------------------ AdamW
// p, m, v fp32 in place; g bf16 or fp32; optional bf16 working copy of the new p.
// bc1 = 1 - b1^t, bc2 = 1 - b2^t (computed on the host in double), or, with hyper_dev, lr and the
// two bias corrections read from device memory (a host whose schedule and step count live on
// the device, like optax's injected hyper-parameters inside a jitted step).
// p - lr (m_hat / (sqrt(v_hat) + eps) + wd p) with the hardware square root and reciprocal (1 ulp
// each) instead of the correctly rounded library forms: those expand to ~22 vector instructions
// per element, and when this kernel shares a CU with a GEMM every vector instruction it issues
// takes an issue slot from the GEMM's MFMAs.  The update moves by a few 1e-7 of its own size
// (lr-sized), far below one ulp of p.
__device__ __forceinline__ float adamw_new_p(float p, float mh, float vh, float lr, float eps, float wd) {
  const float r = __builtin_amdgcn_rcpf(__builtin_amdgcn_sqrtf(vh) + eps);
  return __builtin_fmaf(-lr, __builtin_fmaf(mh, r, wd * p), p);
}

template <bool G_BF16>
__global__ __launch_bounds__(256) __attribute__((amdgpu_num_vgpr(16))) void adamw_kernel(
    float* __restrict__ p, const void* __restrict__ gv, float* __restrict__ m, float* __restrict__ v,
    bf16* __restrict__ shadow, int64_t n, float lr, float b1, float b2, float eps, float wd, float bc1,
    float bc2, float gscale, const float* __restrict__ gscale_dev, const float* __restrict__ hyper_dev) {
  if (gscale_dev) gscale *= *gscale_dev;
  if (hyper_dev) {  // step-dependent scalars from device memory (wave-uniform scalar loads)
    lr = hyper_dev[0];
    bc1 = hyper_dev[1];
    bc2 = hyper_dev[2];
  }
  const int64_t n4 = n / 4;
  const float ibc1 = 1.f / bc1, ibc2 = 1.f / bc2, omb1 = 1.f - b1, omb2 = 1.f - b2;
  // Every element is touched exactly once: streaming (non-temporal) accesses keep the 28 B/param
  // out of the way of the L2.  The kernel is held to 32 registers (amdgpu_num_vgpr counts pairs
  // of the unified file on this target) so that one of its waves fits on a SIMD beside two
  // 240-register GEMM waves when it runs on a second stream, and it is launched as a small
  // grid-stride grid (two workgroups per CU): the whole grid then sweeps five arrays as
  // contiguous 2 MB fronts, which measured 5.6 TB/s against 4.7 TB/s for one workgroup per 8 KB.
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) {
    f32x4 pv = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p) + i);
    f32x4 mv = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(m) + i);
    f32x4 vv = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(v) + i);
    float g[4];
    if (G_BF16) {
      Pack4 gp;
      gp.u = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(gv) + i);
#pragma unroll
      for (int e = 0; e < 4; e++) g[e] = bf2f(gp.e[e]);
    } else {
      f32x4 gf = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(gv) + i);
#pragma unroll
      for (int e = 0; e < 4; e++) g[e] = gf[e];
    }
    Pack4 sh;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const float ge = g[e] * gscale;
      mv[e] = b1 * mv[e] + omb1 * ge;
      vv[e] = b2 * vv[e] + omb2 * ge * ge;
      pv[e] = adamw_new_p(pv[e], mv[e] * ibc1, vv[e] * ibc2, lr, eps, wd);
      sh.e[e] = f2bf(pv[e]);
    }
    __builtin_nontemporal_store(pv, reinterpret_cast<f32x4*>(p) + i);
    __builtin_nontemporal_store(mv, reinterpret_cast<f32x4*>(m) + i);
    __builtin_nontemporal_store(vv, reinterpret_cast<f32x4*>(v) + i);
    if (shadow) __builtin_nontemporal_store(sh.u, reinterpret_cast<u32x2*>(shadow) + i);
  }
  // tail (n % 4) handled by the first threads of block 0
  if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
    const int64_t i = n4 * 4 + threadIdx.x;
    const float ge = (G_BF16 ? bf2f(reinterpret_cast<const bf16*>(gv)[i]) : reinterpret_cast<const float*>(gv)[i]) * gscale;
    // the same operations in the same order as the vector body: where a range is cut does not
    // change any element's result
    const float mm = b1 * m[i] + omb1 * ge;
    const float vv = b2 * v[i] + omb2 * ge * ge;
    const float pp = adamw_new_p(p[i], mm * ibc1, vv * ibc2, lr, eps, wd);
    m[i] = mm;
    v[i] = vv;
    p[i] = pp;
    if (shadow) shadow[i] = f2bf(pp);
  }
}

// sum of squares of a gradient leaf, accumulated (fp32 atomics) into *out
template <bool G_BF16>
__global__ __launch_bounds__(256) void sumsq_kernel(const void* __restrict__ gv, int64_t n,
                                                    float* __restrict__ out) {
  __shared__ float red[4];
  float s = 0.f;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const float g = G_BF16 ? bf2f(reinterpret_cast<const bf16*>(gv)[i]) : reinterpret_cast<const float*>(gv)[i];
    s += g * g;
  }
  s = block_sum<4>(s, red);
  if (threadIdx.x == 0) atomicAdd(out, s);
}

__global__ void cast_f32_bf16_kernel(const float* __restrict__ in, bf16* __restrict__ out, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    out[i] = f2bf(in[i]);
}
__global__ void cast_bf16_f32_kernel(const bf16* __restrict__ in, float* __restrict__ out, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    out[i] = bf2f(in[i]);
}
__global__ void fill_u32_kernel(uint32_t* __restrict__ p, uint32_t val, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    p[i] = val;
}
// out = a + b (bf16), 8 per lane
__global__ __launch_bounds__(256) void add_bf16_kernel(const bf16* __restrict__ a, const bf16* __restrict__ b,
                                                       bf16* __restrict__ out, int64_t n8) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (int64_t)gridDim.x * 256) {
    Pack8 x, y, o;
    x.u = reinterpret_cast<const u32x4*>(a)[i];
    y.u = reinterpret_cast<const u32x4*>(b)[i];
#pragma unroll
    for (int e = 0; e < 8; e++) o.e[e] = f2bf(bf2f(x.e[e]) + bf2f(y.e[e]));
    reinterpret_cast<u32x4*>(out)[i] = o.u;
  }
}

int grid_1d(int64_t items, int cap = 8192) {
  int64_t g = (items + 255) / 256;
  return (int)(g < 1 ? 1 : (g > cap ? cap : g));
}

}  // namespace

extern "C" int32_t olmax_glu_fwd(hipStream_t stream, const void* gate, const void* up, void* out,
                                 int64_t T, int32_t F, int64_t ldg, int64_t ldu, int64_t ldo,
                                 int32_t act) {
  if (T == 0) return OLMAX_OK;
  OLMAX_CHECK(gate && up && out, OLMAX_ERR_ARG, "olmax_glu_fwd: null pointer");
  OLMAX_CHECK(T >= 0 && F > 0 && ldg >= F && ldu >= F && ldo >= F, OLMAX_ERR_SHAPE, "olmax_glu_fwd: bad shape");
  OLMAX_CHECK(act == 0 || act == 1, OLMAX_ERR_ARG, "olmax_glu_fwd: act must be 0 (silu) or 1 (gelu-tanh)");
  const bf16 *g = (const bf16*)gate, *u = (const bf16*)up;
  bf16* o = (bf16*)out;
  const bool vec = F % 8 == 0 && ldg % 8 == 0 && ldu % 8 == 0 && ldo % 8 == 0 && aligned16(gate) && aligned16(up) && aligned16(out);
  if (vec) {
    const int grid = grid_1d(T * (F / 8));
    if (act) hipLaunchKernelGGL(glu_fwd_kernel<true>, dim3(grid), dim3(256), 0, stream, g, u, o, T, F, ldg, ldu, ldo);
    else hipLaunchKernelGGL(glu_fwd_kernel<false>, dim3(grid), dim3(256), 0, stream, g, u, o, T, F, ldg, ldu, ldo);
  } else {
    const unsigned grid = (unsigned)((T * F + 255) / 256);
    if (act) hipLaunchKernelGGL(glu_fwd_scalar<true>, dim3(grid), dim3(256), 0, stream, g, u, o, T, F, ldg, ldu, ldo);
    else hipLaunchKernelGGL(glu_fwd_scalar<false>, dim3(grid), dim3(256), 0, stream, g, u, o, T, F, ldg, ldu, ldo);
  }
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}

extern "C" int32_t olmax_glu_bwd(hipStream_t stream, const void* gate, const void* up,
                                 const void* dh, void* dgate, void* dup, int64_t T, int32_t F,
                                 int64_t ldg, int64_t ldu, int64_t lddh, int64_t lddg, int64_t lddu,
                                 int32_t act) {
  if (T == 0) return OLMAX_OK;
  OLMAX_CHECK(gate && up && dh && dgate && dup, OLMAX_ERR_ARG, "olmax_glu_bwd: null pointer");
  OLMAX_CHECK(T >= 0 && F > 0 && ldg >= F && ldu >= F && lddh >= F && lddg >= F && lddu >= F, OLMAX_ERR_SHAPE, "olmax_glu_bwd: bad shape");
  OLMAX_CHECK(act == 0 || act == 1, OLMAX_ERR_ARG, "olmax_glu_bwd: act must be 0 (silu) or 1 (gelu-tanh)");
  const bf16 *g = (const bf16*)gate, *u = (const bf16*)up, *d = (const bf16*)dh;
  bf16 *og = (bf16*)dgate, *ou = (bf16*)dup;
  const bool vec = F % 8 == 0 && ldg % 8 == 0 && ldu % 8 == 0 && lddh % 8 == 0 && lddg % 8 == 0 && lddu % 8 == 0 &&
                   aligned16(gate) && aligned16(up) && aligned16(dh) && aligned16(dgate) && aligned16(dup);
  if (vec) {
    const int grid = grid_1d(T * (F / 8));
    if (act) hipLaunchKernelGGL(glu_bwd_kernel<true>, dim3(grid), dim3(256), 0, stream, g, u, d, og, ou, T, F, ldg, ldu, lddh, lddg, lddu);
    else hipLaunchKernelGGL(glu_bwd_kernel<false>, dim3(grid), dim3(256), 0, stream, g, u, d, og, ou, T, F, ldg, ldu, lddh, lddg, lddu);
  } else {
    const unsigned grid = (unsigned)((T * F + 255) / 256);
    if (act) hipLaunchKernelGGL(glu_bwd_scalar<true>, dim3(grid), dim3(256), 0, stream, g, u, d, og, ou, T, F, ldg, ldu, lddh, lddg, lddu);
    else hipLaunchKernelGGL(glu_bwd_scalar<false>, dim3(grid), dim3(256), 0, stream, g, u, d, og, ou, T, F, ldg, ldu, lddh, lddg, lddu);
  }
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}

extern "C" int32_t olmax_embed_fwd(hipStream_t stream, const int32_t* ids, const void* W, void* out,
                                   int64_t T, int32_t d, int32_t V) {
  if (T == 0) return OLMAX_OK;
  OLMAX_CHECK(ids && W && out, OLMAX_ERR_ARG, "olmax_embed_fwd: null pointer");
  OLMAX_CHECK(T >= 0 && d > 0 && V > 0, OLMAX_ERR_SHAPE, "olmax_embed_fwd: bad shape");
  if (d % 8 == 0 && aligned16(W) && aligned16(out))
    hipLaunchKernelGGL(embed_fwd_kernel, dim3(grid_1d(T * (d / 8))), dim3(256), 0, stream, ids, (const bf16*)W, (bf16*)out, T, d, V);
  else
    hipLaunchKernelGGL(embed_fwd_scalar, dim3((unsigned)((T * d + 255) / 256)), dim3(256), 0, stream, ids, (const bf16*)W, (bf16*)out, T, d, V);
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}

extern "C" int32_t olmax_grad_accumulate(hipStream_t stream, float* acc, const void* g, int64_t n, int32_t grad_is_bf16,
                                         int32_t mini_step) {
  if (n == 0) return OLMAX_OK;
  OLMAX_CHECK(acc && g && n >= 0 && mini_step >= 0, OLMAX_ERR_ARG, "olmax_grad_accumulate: bad argument");
  OLMAX_CHECK(aligned16(acc) && (((uintptr_t)g) & (grad_is_bf16 ? 7 : 15)) == 0, OLMAX_ERR_ALIGN,
              "olmax_grad_accumulate: acc / fp32 g must be 16-byte aligned, bf16 g 8-byte aligned");
  const int grid = grid_1d((n + 3) / 4, 2048);
  const float inv = 1.f / (float)(mini_step + 1);
  if (grad_is_bf16) hipLaunchKernelGGL(grad_accum_kernel<true>, dim3(grid), dim3(256), 0, stream, acc, g, n, inv, mini_step == 0);
  else hipLaunchKernelGGL(grad_accum_kernel<false>, dim3(grid), dim3(256), 0, stream, acc, g, n, inv, mini_step == 0);
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}

extern "C" int32_t olmax_sequential_tokens(hipStream_t stream, const int32_t* start_offsets, int32_t* inputs,
                                           int32_t* targets, int32_t B, int32_t S, int32_t V) {
  if (B == 0 || S == 0) return OLMAX_OK;
  OLMAX_CHECK(start_offsets && inputs && targets, OLMAX_ERR_ARG, "olmax_sequential_tokens: null pointer");
  OLMAX_CHECK(B > 0 && S > 0 && V > 0, OLMAX_ERR_SHAPE, "olmax_sequential_tokens: bad shape");
  hipLaunchKernelGGL(sequential_tokens_kernel, dim3(grid_1d((int64_t)B * S)), dim3(256), 0, stream, start_offsets, inputs,
                     targets, B, S, V);
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}

// dW (fp32 [V, d]) is ACCUMULATED into: the caller zeroes it (or seeds it, for tied heads).
extern "C" int32_t olmax_embed_bwd(hipStream_t stream, const int32_t* ids, const void* dh, float* dW,
                                   int64_t T, int32_t d, int32_t V) {
  if (T == 0) return OLMAX_OK;
  OLMAX_CHECK(ids && dh && dW, OLMAX_ERR_ARG, "olmax_embed_bwd: null pointer");
  OLMAX_CHECK(T >= 0 && d > 0 && V > 0, OLMAX_ERR_SHAPE, "olmax_embed_bwd: bad shape");
  hipLaunchKernelGGL(embed_bwd_kernel, dim3(grid_1d(T * d)), dim3(256), 0, stream, ids, (const bf16*)dh, dW, T, d, V);
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}

// As olmax_adamw, with an additional device-resident gradient scale (NULL = none) so that
// global-norm clipping needs no host round trip.
extern "C" int32_t olmax_adamw_dscale(hipStream_t stream, float* p, const void* g, float* m, float* v,
                                      void* shadow_bf16, int64_t n, int32_t grad_is_bf16, float lr, float b1,
                                      float b2, float eps, float wd, int64_t step, float grad_scale,
                                      const float* grad_scale_dev) {
  // two workgroups per CU: the fastest grid when the kernel has the GPU to itself
  return olmax_adamw_grid(stream, p, g, m, v, shadow_bf16, n, grad_is_bf16, lr, b1, b2, eps, wd, step, grad_scale,
                          grad_scale_dev, 512, nullptr);
}

// As olmax_adamw_dscale with lr and the bias corrections in device memory:
// hyper_dev = {lr, 1 - b1^step, 1 - b2^step} (fp32), written by earlier work on the same stream.
extern "C" int32_t olmax_adamw_dev(hipStream_t stream, float* p, const void* g, float* m, float* v, void* shadow_bf16,
                                   int64_t n, int32_t grad_is_bf16, float b1, float b2, float eps, float wd,
                                   const float* hyper_dev, const float* grad_scale_dev) {
  OLMAX_CHECK(hyper_dev, OLMAX_ERR_ARG, "olmax_adamw_dev: hyper_dev is null");
  return olmax_adamw_grid(stream, p, g, m, v, shadow_bf16, n, grad_is_bf16, 0.f, b1, b2, eps, wd, 1, 1.f, grad_scale_dev, 512,
                          hyper_dev);
}

// Library-internal form with the grid size exposed: the overlapped train step runs it with one
// workgroup per CU on its second stream, which disturbs the GEMMs it shares the GPU with least.
int olmax_adamw_grid(hipStream_t stream, float* p, const void* g, float* m, float* v, void* shadow_bf16, int64_t n,
                     int32_t grad_is_bf16, float lr, float b1, float b2, float eps, float wd, int64_t step,
                     float grad_scale, const float* grad_scale_dev, int grid_cap, const float* hyper_dev) {
  if (n == 0) return OLMAX_OK;
  OLMAX_CHECK(p && g && m && v, OLMAX_ERR_ARG, "olmax_adamw: null pointer");
  OLMAX_CHECK(n >= 0 && step >= 1, OLMAX_ERR_ARG, "olmax_adamw: n must be >= 0 and step >= 1 (1-based)");
  OLMAX_CHECK(aligned16(p) && aligned16(m) && aligned16(v) && (((uintptr_t)g) & (grad_is_bf16 ? 7 : 15)) == 0 &&
                  (!shadow_bf16 || (((uintptr_t)shadow_bf16) & 7) == 0),
              OLMAX_ERR_ALIGN, "olmax_adamw: buffers must be 16-byte aligned (bf16 buffers 8-byte)");
  const float bc1 = (float)(1.0 - pow((double)b1, (double)step));
  const float bc2 = (float)(1.0 - pow((double)b2, (double)step));
  const int grid = grid_1d((n + 3) / 4, grid_cap);
  if (grad_is_bf16)
    hipLaunchKernelGGL(adamw_kernel<true>, dim3(grid), dim3(256), 0, stream, p, g, m, v, (bf16*)shadow_bf16, n, lr, b1, b2, eps, wd, bc1, bc2, grad_scale, grad_scale_dev, hyper_dev);
  else
    hipLaunchKernelGGL(adamw_kernel<false>, dim3(grid), dim3(256), 0, stream, p, g, m, v, (bf16*)shadow_bf16, n, lr, b1, b2, eps, wd, bc1, bc2, grad_scale, grad_scale_dev, hyper_dev);
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}

extern "C" int32_t olmax_adamw(hipStream_t stream, float* p, const void* g, float* m, float* v,
                               void* shadow_bf16, int64_t n, int32_t grad_is_bf16, float lr, float b1,
                               float b2, float eps, float wd, int64_t step, float grad_scale) {
  return olmax_adamw_dscale(stream, p, g, m, v, shadow_bf16, n, grad_is_bf16, lr, b1, b2, eps, wd, step, grad_scale, nullptr);
}

// *out (fp32 scalar) += sum(g^2); the caller zeroes it.
extern "C" int32_t olmax_sumsq(hipStream_t stream, const void* g, int64_t n, int32_t is_bf16, float* out) {
  if (n == 0) return OLMAX_OK;
  OLMAX_CHECK(g && out && n >= 0, OLMAX_ERR_ARG, "olmax_sumsq: bad argument");
  const int grid = grid_1d(n, 2048);
  if (is_bf16) hipLaunchKernelGGL(sumsq_kernel<true>, dim3(grid), dim3(256), 0, stream, g, n, out);
  else hipLaunchKernelGGL(sumsq_kernel<false>, dim3(grid), dim3(256), 0, stream, g, n, out);
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}

extern "C" int32_t olmax_cast_f32_to_bf16(hipStream_t stream, const float* in, void* out, int64_t n) {
  if (n == 0) return OLMAX_OK;
  OLMAX_CHECK(in && out && n >= 0, OLMAX_ERR_ARG, "olmax_cast_f32_to_bf16: bad argument");
  hipLaunchKernelGGL(cast_f32_bf16_kernel, dim3(grid_1d(n)), dim3(256), 0, stream, in, (bf16*)out, n);
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}
extern "C" int32_t olmax_cast_bf16_to_f32(hipStream_t stream, const void* in, float* out, int64_t n) {
  if (n == 0) return OLMAX_OK;
  OLMAX_CHECK(in && out && n >= 0, OLMAX_ERR_ARG, "olmax_cast_bf16_to_f32: bad argument");
  hipLaunchKernelGGL(cast_bf16_f32_kernel, dim3(grid_1d(n)), dim3(256), 0, stream, (const bf16*)in, out, n);
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}
// Fill kernel (graph-capture safe replacement for memset); nbytes must be a multiple of 4.
extern "C" int32_t olmax_fill_zero(hipStream_t stream, void* p, int64_t nbytes) {
  OLMAX_CHECK(p && nbytes >= 0 && nbytes % 4 == 0 && (((uintptr_t)p) & 3) == 0, OLMAX_ERR_ARG, "olmax_fill_zero: need 4-byte aligned pointer and size");
  if (nbytes == 0) return OLMAX_OK;
  hipLaunchKernelGGL(fill_u32_kernel, dim3(grid_1d(nbytes / 4)), dim3(256), 0, stream, (uint32_t*)p, 0u, nbytes / 4);
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}
extern "C" int32_t olmax_add_bf16(hipStream_t stream, const void* a, const void* b, void* out, int64_t n) {
  if (n == 0) return OLMAX_OK;
  OLMAX_CHECK(a && b && out && n >= 0 && n % 8 == 0 && aligned16(a) && aligned16(b) && aligned16(out), OLMAX_ERR_ARG, "olmax_add_bf16: need n % 8 == 0 and 16-byte alignment");
  hipLaunchKernelGGL(add_bf16_kernel, dim3(grid_1d(n / 8)), dim3(256), 0, stream, (const bf16*)a, (const bf16*)b, (bf16*)out, n / 8);
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}
