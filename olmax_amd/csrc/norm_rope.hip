// HBM-bound row kernels: RMSNorm forward/backward and the fused head-wise QK-norm + RoPE
// forward/backward.  All of them move 128 bits per lane per access and reduce rows with
// wave64 xor-shuffles; statistics and arithmetic are fp32, storage bf16.
//
// Reference semantics:
//   rms_norm            src/olmax/nn/functional.py:51-67  (fp32 internally, cast back)
//   head-wise QK-norm   src/olmax/nn/attention.py:293-296 (one [head_dim] weight for all heads)
//   RoPE                src/olmax/nn/rope.py:62-65,99-115 (rotate_half pairing i <-> i + D/2)
#include "common.h"

namespace {


// ------------------------------------------------------------------ RMSNorm forward
// LPR lanes cooperate on one row; a 256-thread block handles 256/LPR rows per iteration.
template <int LPR, int MAXC>
__global__ __launch_bounds__(256) void rmsnorm_fwd_kernel(const bf16* __restrict__ x,
                                                          const bf16* __restrict__ w,
                                                          const bf16* __restrict__ res,
                                                          bf16* __restrict__ y, int64_t rows, int d,
                                                          int64_t ldx, int64_t ldres, int64_t ldy,
                                                          float eps) {
  constexpr int RPB = 256 / LPR;
  const int sub = threadIdx.x % LPR;
  const int rloc = threadIdx.x / LPR;
  for (int64_t row = (int64_t)blockIdx.x * RPB + rloc; row < rows; row += (int64_t)gridDim.x * RPB) {
    const bf16* xr = x + row * ldx;
    Pack8 c[MAXC];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < MAXC; i++)
      if ((i * LPR + sub) * 8 < d) {
        c[i].u = *reinterpret_cast<const u32x4*>(xr + (i * LPR + sub) * 8);
#pragma unroll
        for (int e = 0; e < 8; e++) {
          const float f = bf2f(c[i].e[e]);
          ss += f * f;
        }
      }
#pragma unroll
    for (int o = LPR / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    const float r = rsqrtf(ss / (float)d + eps);
    bf16* yr = y + row * ldy;
#pragma unroll
    for (int i = 0; i < MAXC; i++)
      if ((i * LPR + sub) * 8 < d) {
        Pack8 wv, rv, o;
        if (w) wv.u = *reinterpret_cast<const u32x4*>(w + (i * LPR + sub) * 8);
        if (res) rv.u = *reinterpret_cast<const u32x4*>(res + row * ldres + (i * LPR + sub) * 8);
#pragma unroll
        for (int e = 0; e < 8; e++) {
          float v = r * bf2f(c[i].e[e]);
          if (w) v = bf2f(wv.e[e]) * v;
          if (res) v = bf2f(f2bf(v)) + bf2f(rv.e[e]);  // the reference adds two bf16 arrays
          o.e[e] = f2bf(v);
        }
        *reinterpret_cast<u32x4*>(yr + (i * LPR + sub) * 8) = o.u;
      }
  }
}

// Any d (scalar accesses, one block per row): used for odd row lengths.
__global__ __launch_bounds__(256) void rmsnorm_fwd_generic(const bf16* __restrict__ x,
                                                           const bf16* __restrict__ w,
                                                           const bf16* __restrict__ res,
                                                           bf16* __restrict__ y, int64_t rows, int d,
                                                           int64_t ldx, int64_t ldres, int64_t ldy,
                                                           float eps) {
  __shared__ float red[4];
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const bf16* xr = x + row * ldx;
    float ss = 0.f;
    for (int i = threadIdx.x; i < d; i += 256) {
      const float f = bf2f(xr[i]);
      ss += f * f;
    }
    ss = block_sum<4>(ss, red);
    const float r = rsqrtf(ss / (float)d + eps);
    for (int i = threadIdx.x; i < d; i += 256) {
      float v = r * bf2f(xr[i]);
      if (w) v = bf2f(w[i]) * v;
      if (res) v = bf2f(f2bf(v)) + bf2f(res[row * ldres + i]);
      y[row * ldy + i] = f2bf(v);
    }
    __syncthreads();
  }
}

// ------------------------------------------------------------------ RMSNorm backward
// dx = r*g - x * r^3 * mean(x*g), g = w*dy;   dw[c] += sum_rows dy*x*r   (fp32 atomics)
// Optional `dres` is added to dx (fused residual-gradient add).
// Narrow rows (d <= 1024): LPR lanes of one wave own a row, which stays in registers between the
// two passes, and the lanes' columns sums live in registers until the end.
template <int LPR, int MAXC, int THREADS>
__global__ __launch_bounds__(THREADS) void rmsnorm_bwd_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ w, const bf16* __restrict__ dy,
    const bf16* __restrict__ dres, bf16* __restrict__ dx, float* __restrict__ dw, int64_t rows,
    int d, int64_t ldx, int64_t lddy, int64_t lddres, int64_t lddx, float eps) {
  constexpr int RPB = THREADS / LPR;
  const int sub = threadIdx.x % LPR;
  const int rloc = threadIdx.x / LPR;
  float dwacc[MAXC][8];
#pragma unroll
  for (int i = 0; i < MAXC; i++)
#pragma unroll
    for (int e = 0; e < 8; e++) dwacc[i][e] = 0.f;

  for (int64_t row = (int64_t)blockIdx.x * RPB + rloc; row < rows; row += (int64_t)gridDim.x * RPB) {
    const bf16* xr = x + row * ldx;
    const bf16* dyr = dy + row * lddy;
    Pack8 cx[MAXC], cg[MAXC];
    float ss = 0.f, sxg = 0.f;
#pragma unroll
    for (int i = 0; i < MAXC; i++)
      if ((i * LPR + sub) * 8 < d) {
        cx[i].u = *reinterpret_cast<const u32x4*>(xr + (i * LPR + sub) * 8);
        cg[i].u = *reinterpret_cast<const u32x4*>(dyr + (i * LPR + sub) * 8);
        Pack8 wv;
        if (w) wv.u = *reinterpret_cast<const u32x4*>(w + (i * LPR + sub) * 8);
#pragma unroll
        for (int e = 0; e < 8; e++) {
          const float xf = bf2f(cx[i].e[e]);
          const float g = w ? bf2f(wv.e[e]) * bf2f(cg[i].e[e]) : bf2f(cg[i].e[e]);
          ss += xf * xf;
          sxg += xf * g;
        }
      }
#pragma unroll
    for (int o = LPR / 2; o > 0; o >>= 1) {
      ss += __shfl_xor(ss, o, 64);
      sxg += __shfl_xor(sxg, o, 64);
    }
    const float r = rsqrtf(ss / (float)d + eps);
    const float coef = r * r * r * (sxg / (float)d);
    bf16* dxr = dx + row * lddx;
#pragma unroll
    for (int i = 0; i < MAXC; i++)
      if ((i * LPR + sub) * 8 < d) {
        Pack8 wv, rv, o;
        if (w) wv.u = *reinterpret_cast<const u32x4*>(w + (i * LPR + sub) * 8);
        if (dres) rv.u = *reinterpret_cast<const u32x4*>(dres + row * lddres + (i * LPR + sub) * 8);
#pragma unroll
        for (int e = 0; e < 8; e++) {
          const float xf = bf2f(cx[i].e[e]);
          const float dyf = bf2f(cg[i].e[e]);
          const float g = w ? bf2f(wv.e[e]) * dyf : dyf;
          float v = r * g - xf * coef;
          if (dres) v = bf2f(f2bf(v)) + bf2f(rv.e[e]);  // the reference adds two bf16 arrays
          o.e[e] = f2bf(v);
          dwacc[i][e] += dyf * xf * r;
        }
        *reinterpret_cast<u32x4*>(dxr + (i * LPR + sub) * 8) = o.u;
      }
  }
  if (dw) {
    // Combine the RPB row-slots of this block in LDS, then one global atomic per column per
    // block.  Global fp32 atomics are the expensive part (they are resolved beyond the per-XCD
    // L2s, ~50 G/s), so the launch uses few, fat blocks; inside the block the slots add in turn
    // (each lane owns its columns, so plain read-modify-write is enough).
    extern __shared__ float sdw[];  // d floats
#pragma unroll 1
    for (int turn = 0; turn < RPB; turn++) {
      if (rloc == turn) {
#pragma unroll
        for (int i = 0; i < MAXC; i++)
          if ((i * LPR + sub) * 8 < d) {
            float* dst = &sdw[(i * LPR + sub) * 8];
            f32x4 lo, hi;
            if (turn == 0) {
#pragma unroll
              for (int e = 0; e < 4; e++) { lo[e] = dwacc[i][e]; hi[e] = dwacc[i][4 + e]; }
            } else {
              lo = *reinterpret_cast<f32x4*>(dst);
              hi = *reinterpret_cast<f32x4*>(dst + 4);
#pragma unroll
              for (int e = 0; e < 4; e++) { lo[e] += dwacc[i][e]; hi[e] += dwacc[i][4 + e]; }
            }
            *reinterpret_cast<f32x4*>(dst) = lo;
            *reinterpret_cast<f32x4*>(dst + 4) = hi;
          }
      }
      __syncthreads();
    }
    for (int i = threadIdx.x; i < d; i += THREADS) atomicAdd(&dw[i], sdw[i]);
  }
}

// Wide rows (2048 < d <= 8192).  WPR waves share one row, a lane owns MAXC chunks of 8 columns,
// so the row held between the two passes and the dw column sums take 12 * MAXC registers
// instead of 128 + 64: sixteen waves fit on a CU, and for a kernel that only streams, waves in
// flight are what sets the bandwidth.  The waves of a row exchange their partial sums through
// LDS (two slots used in turn, one barrier per iteration); the next row's x, dy and dres are
// already on their way while the current one is reduced.
template <int WPR, int MAXC, int THREADS>
__global__ __launch_bounds__(THREADS) void rmsnorm_bwd_split_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ w, const bf16* __restrict__ dy,
    const bf16* __restrict__ dres, bf16* __restrict__ dx, float* __restrict__ dw, int64_t rows,
    int d, int64_t ldx, int64_t lddy, int64_t lddres, int64_t lddx, float eps) {
  constexpr int RPB = THREADS / (64 * WPR);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rloc = wave / WPR, part = wave % WPR;
  __shared__ float red[2][RPB][WPR][2];
  extern __shared__ float sdw[];  // d floats when dw is asked for

  int col[MAXC];
  bool on[MAXC];
  Pack8 wv[MAXC];
  float dwacc[MAXC][8];
#pragma unroll
  for (int i = 0; i < MAXC; i++) {
    col[i] = ((i * WPR + part) * 64 + lane) * 8;
    on[i] = col[i] < d;
    wv[i].u = {0u, 0u, 0u, 0u};  // lanes past the end of the row contribute exact zeros
    if (w && on[i]) wv[i].u = *reinterpret_cast<const u32x4*>(w + col[i]);
#pragma unroll
    for (int e = 0; e < 8; e++) dwacc[i][e] = 0.f;
  }
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  Pack8 nx[MAXC], ng[MAXC], nr[MAXC];
  auto fetch = [&](int64_t row) {
    if (row < rows) {
#pragma unroll
      for (int i = 0; i < MAXC; i++)
        if (on[i]) {
          nx[i].u = *reinterpret_cast<const u32x4*>(x + row * ldx + col[i]);
          ng[i].u = *reinterpret_cast<const u32x4*>(dy + row * lddy + col[i]);
          if (dres) nr[i].u = *reinterpret_cast<const u32x4*>(dres + row * lddres + col[i]);
        }
    }
  };
  const int64_t step = (int64_t)gridDim.x * RPB;
  int64_t base = (int64_t)blockIdx.x * RPB;
  fetch(base + rloc);
  int buf = 0;
  for (; base < rows; base += step, buf ^= 1) {
    const int64_t row = base + rloc;
    Pack8 cx[MAXC], cg[MAXC], cr[MAXC];
#pragma unroll
    for (int i = 0; i < MAXC; i++) {
      cx[i].u = on[i] ? nx[i].u : zero4;
      cg[i].u = on[i] ? ng[i].u : zero4;
      cr[i].u = nr[i].u;
    }
    fetch(row + step);
    float ss = 0.f, sxg = 0.f;
#pragma unroll
    for (int i = 0; i < MAXC; i++)
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const float xf = bf2f(cx[i].e[e]);
        const float g = w ? bf2f(wv[i].e[e]) * bf2f(cg[i].e[e]) : bf2f(cg[i].e[e]);
        ss += xf * xf;
        sxg += xf * g;
      }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      ss += __shfl_xor(ss, o, 64);
      sxg += __shfl_xor(sxg, o, 64);
    }
    if (lane == 0) {
      red[buf][rloc][part][0] = ss;
      red[buf][rloc][part][1] = sxg;
    }
    __syncthreads();
    // Keep the row packed across the barrier: without this the compiler carries the widened
    // floats of the first pass into the second and doubles the register count.
#pragma unroll
    for (int i = 0; i < MAXC; i++) {
      asm volatile("" : "+v"(cx[i].u), "+v"(cg[i].u), "+v"(wv[i].u));
    }
    ss = 0.f;
    sxg = 0.f;
#pragma unroll
    for (int p = 0; p < WPR; p++) {
      ss += red[buf][rloc][p][0];
      sxg += red[buf][rloc][p][1];
    }
    if (row < rows) {
      const float r = rsqrtf(ss / (float)d + eps);
      const float coef = r * r * r * (sxg / (float)d);
#pragma unroll
      for (int i = 0; i < MAXC; i++)
        if (on[i]) {
          Pack8 o;
#pragma unroll
          for (int e = 0; e < 8; e++) {
            const float xf = bf2f(cx[i].e[e]);
            const float dyf = bf2f(cg[i].e[e]);
            const float g = w ? bf2f(wv[i].e[e]) * dyf : dyf;
            float v = r * g - xf * coef;
            if (dres) v = bf2f(f2bf(v)) + bf2f(cr[i].e[e]);  // the reference adds two bf16 arrays
            o.e[e] = f2bf(v);
            dwacc[i][e] += dyf * xf * r;
          }
          *reinterpret_cast<u32x4*>(dx + row * lddx + col[i]) = o.u;
        }
    }
  }
  if (dw) {
    // The RPB row slots of the block add their column sums in LDS in turn (every column has one
    // owner per slot), then one global atomic per column and block.
#pragma unroll 1
    for (int turn = 0; turn < RPB; turn++) {
      if (rloc == turn) {
#pragma unroll
        for (int i = 0; i < MAXC; i++)
          if (on[i]) {
            float* dst = &sdw[col[i]];
            f32x4 lo, hi;
            if (turn == 0) {
#pragma unroll
              for (int e = 0; e < 4; e++) { lo[e] = dwacc[i][e]; hi[e] = dwacc[i][4 + e]; }
            } else {
              lo = *reinterpret_cast<f32x4*>(dst);
              hi = *reinterpret_cast<f32x4*>(dst + 4);
#pragma unroll
              for (int e = 0; e < 4; e++) { lo[e] += dwacc[i][e]; hi[e] += dwacc[i][4 + e]; }
            }
            *reinterpret_cast<f32x4*>(dst) = lo;
            *reinterpret_cast<f32x4*>(dst + 4) = hi;
          }
      }
      __syncthreads();
    }
    for (int i = threadIdx.x; i < d; i += THREADS) atomicAdd(&dw[i], sdw[i]);
  }
}

__global__ __launch_bounds__(256) void rmsnorm_bwd_generic(
    const bf16* __restrict__ x, const bf16* __restrict__ w, const bf16* __restrict__ dy,
    const bf16* __restrict__ dres, bf16* __restrict__ dx, float* __restrict__ dw, int64_t rows,
    int d, int64_t ldx, int64_t lddy, int64_t lddres, int64_t lddx, float eps) {
  __shared__ float red[4];
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    const bf16* xr = x + row * ldx;
    const bf16* dyr = dy + row * lddy;
    float ss = 0.f, sxg = 0.f;
    for (int i = threadIdx.x; i < d; i += 256) {
      const float xf = bf2f(xr[i]);
      const float g = w ? bf2f(w[i]) * bf2f(dyr[i]) : bf2f(dyr[i]);
      ss += xf * xf;
      sxg += xf * g;
    }
    ss = block_sum<4>(ss, red);
    sxg = block_sum<4>(sxg, red);
    const float r = rsqrtf(ss / (float)d + eps);
    const float coef = r * r * r * (sxg / (float)d);
    for (int i = threadIdx.x; i < d; i += 256) {
      const float xf = bf2f(xr[i]);
      const float dyf = bf2f(dyr[i]);
      const float g = w ? bf2f(w[i]) * dyf : dyf;
      float v = r * g - xf * coef;
      if (dres) v = bf2f(f2bf(v)) + bf2f(dres[row * lddres + i]);
      dx[row * lddx + i] = f2bf(v);
      if (dw) atomicAdd(&dw[i], dyf * xf * r);
    }
    __syncthreads();
  }
}

// ------------------------------------------------------------------ QK-norm + RoPE
// One 16-lane group per (token, head) row of D = 128 elements (8 per lane); lanes j and j^8
// hold the rotate_half partners (i, i + 64).  `pos = token % seq_len`.
// Forward:  y = rope( w * (x * rsqrt(mean x^2 + eps)) )   (norm part skipped when w == nullptr;
//           the normalised value is rounded to bf16 before the rotation, as two reference ops)
template <bool NORM>
__global__ __launch_bounds__(256) void qk_rope_fwd_kernel(
    const bf16* __restrict__ x, bf16* __restrict__ y, const bf16* __restrict__ w,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int64_t tokens, int heads,
    int seq_len, int64_t ldx, int64_t ldy, float eps) {
  const int sub = threadIdx.x & 15;
  const int64_t unit = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 4;
  if (unit >= tokens * heads) return;
  const int64_t tok = unit / heads;
  const int h = (int)(unit % heads);
  const int pos = (int)(tok % seq_len);
  Pack8 c;
  c.u = *reinterpret_cast<const u32x4*>(x + tok * ldx + h * 128 + sub * 8);
  float v[8];
#pragma unroll
  for (int e = 0; e < 8; e++) v[e] = bf2f(c.e[e]);
  if (NORM) {
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) ss += v[e] * v[e];
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    const float r = rsqrtf(ss / 128.f + eps);
    Pack8 wv;
    wv.u = *reinterpret_cast<const u32x4*>(w + sub * 8);
#pragma unroll
    for (int e = 0; e < 8; e++) v[e] = bf2f(f2bf(bf2f(wv.e[e]) * (r * v[e])));
  }
  // partner values (lane ^ 8): elements i+64 for sub < 8, i-64 otherwise
  const int fi = (sub & 7) * 8;  // frequency index of this lane's first element
  const float sign = sub < 8 ? -1.f : 1.f;
  Pack8 o;
#pragma unroll
  for (int e = 0; e < 8; e++) {
    const float pv = __shfl_xor(v[e], 8, 64);
    const float cs = cos_t[(int64_t)pos * 64 + fi + e];
    const float sn = sin_t[(int64_t)pos * 64 + fi + e];
    o.e[e] = f2bf(v[e] * cs + sign * pv * sn);
  }
  *reinterpret_cast<u32x4*>(y + tok * ldy + h * 128 + sub * 8) = o.u;
}

// Backward: dr = rope^T(dy) (rotation by -angle, rounded to bf16), then, if NORM, the RMSNorm
// backward against the raw projection x; dw[128] accumulated with fp32 atomics.
template <bool NORM>
__global__ __launch_bounds__(256) void qk_rope_bwd_kernel(
    const bf16* __restrict__ dy, bf16* __restrict__ dx, const bf16* __restrict__ x,
    const bf16* __restrict__ w, float* __restrict__ dw, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int64_t tokens, int heads, int seq_len, int64_t lddy,
    int64_t lddx, int64_t ldx, float eps) {
  __shared__ float sdw[128];
  if (NORM) {
    if (threadIdx.x < 128) sdw[threadIdx.x] = 0.f;
    __syncthreads();
  }
  const int sub = threadIdx.x & 15;
  // a thread always serves the same 8 head-dim columns: its weight-gradient partials stay in
  // registers over the grid-stride loop (few blocks, so few global atomics on the 128 addresses)
  float dwacc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const int64_t units = tokens * heads;
  for (int64_t unit = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4); unit < units; unit += (int64_t)gridDim.x * 16) {
    const int64_t tok = unit / heads;
    const int h = (int)(unit % heads);
    const int pos = (int)(tok % seq_len);
    Pack8 c;
    c.u = *reinterpret_cast<const u32x4*>(dy + tok * lddy + h * 128 + sub * 8);
    const int fi = (sub & 7) * 8;
    const float sign = sub < 8 ? 1.f : -1.f;
    float g[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const float dv = bf2f(c.e[e]);
      const float pv = __shfl_xor(dv, 8, 64);
      const float cs = cos_t[(int64_t)pos * 64 + fi + e];
      const float sn = sin_t[(int64_t)pos * 64 + fi + e];
      g[e] = dv * cs + sign * pv * sn;
    }
    Pack8 o;
    if (NORM) {
      Pack8 xv, wv;
      xv.u = *reinterpret_cast<const u32x4*>(x + tok * ldx + h * 128 + sub * 8);
      wv.u = *reinterpret_cast<const u32x4*>(w + sub * 8);
      float ss = 0.f, sxg = 0.f;
      float xf[8], gg[8];
#pragma unroll
      for (int e = 0; e < 8; e++) {
        g[e] = bf2f(f2bf(g[e]));
        xf[e] = bf2f(xv.e[e]);
        gg[e] = bf2f(wv.e[e]) * g[e];
        ss += xf[e] * xf[e];
        sxg += xf[e] * gg[e];
      }
#pragma unroll
      for (int s = 8; s > 0; s >>= 1) {
        ss += __shfl_xor(ss, s, 64);
        sxg += __shfl_xor(sxg, s, 64);
      }
      const float r = rsqrtf(ss / 128.f + eps);
      const float coef = r * r * r * (sxg / 128.f);
#pragma unroll
      for (int e = 0; e < 8; e++) {
        o.e[e] = f2bf(r * gg[e] - xf[e] * coef);
        dwacc[e] += g[e] * xf[e] * r;
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; e++) o.e[e] = f2bf(g[e]);
    }
    *reinterpret_cast<u32x4*>(dx + tok * lddx + h * 128 + sub * 8) = o.u;
  }
  if (NORM) {
#pragma unroll
    for (int e = 0; e < 8; e++) atomicAdd(&sdw[sub * 8 + e], dwacc[e]);
    __syncthreads();
    if (threadIdx.x < 128) atomicAdd(&dw[threadIdx.x], sdw[threadIdx.x]);
  }
}

// Any even head_dim <= 512, strided views: one wave per (token, head); lane i handles rotation
// pairs (i, i + D/2), (i + 64, ...).  Optional fused head-wise norm, same rounding as above.
__global__ __launch_bounds__(64) void qk_rope_fwd_generic(
    const bf16* __restrict__ x, bf16* __restrict__ y, const bf16* __restrict__ w,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int64_t tokens, int heads, int D,
    int seq_len, int64_t ldx, int64_t ldy, float eps) {
  const int64_t unit = blockIdx.x;
  const int64_t tok = unit / heads;
  const int h = (int)(unit % heads);
  const int pos = (int)(tok % seq_len);
  const int half = D / 2;
  const bf16* xr = x + tok * ldx + h * D;
  bf16* yr = y + tok * ldy + h * D;
  float r = 1.f;
  if (w) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < D; i += 64) {
      const float f = bf2f(xr[i]);
      ss += f * f;
    }
    ss = wave_sum(ss);
    r = rsqrtf(ss / (float)D + eps);
  }
  for (int i = threadIdx.x; i < half; i += 64) {
    float a = bf2f(xr[i]), b = bf2f(xr[i + half]);
    if (w) {
      a = bf2f(f2bf(bf2f(w[i]) * (r * a)));
      b = bf2f(f2bf(bf2f(w[i + half]) * (r * b)));
    }
    const float cs = cos_t[(int64_t)pos * half + i], sn = sin_t[(int64_t)pos * half + i];
    yr[i] = f2bf(a * cs - b * sn);
    yr[i + half] = f2bf(b * cs + a * sn);
  }
}

__global__ __launch_bounds__(64) void qk_rope_bwd_generic(
    const bf16* __restrict__ dy, bf16* __restrict__ dx, const bf16* __restrict__ x,
    const bf16* __restrict__ w, float* __restrict__ dw, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int64_t tokens, int heads, int D, int seq_len, int64_t lddy,
    int64_t lddx, int64_t ldx, float eps) {
  const int64_t unit = blockIdx.x;
  const int64_t tok = unit / heads;
  const int h = (int)(unit % heads);
  const int pos = (int)(tok % seq_len);
  const int half = D / 2;
  const bf16* dyr = dy + tok * lddy + h * D;
  bf16* dxr = dx + tok * lddx + h * D;
  // each lane owns pairs i = lane, lane+64, ... (at most 4 pairs for D <= 512)
  float ga[4], gb[4];
  int np = 0;
  for (int i = threadIdx.x; i < half; i += 64, np++) {
    const float d1 = bf2f(dyr[i]), d2 = bf2f(dyr[i + half]);
    const float cs = cos_t[(int64_t)pos * half + i], sn = sin_t[(int64_t)pos * half + i];
    ga[np] = d1 * cs + d2 * sn;
    gb[np] = d2 * cs - d1 * sn;
  }
  if (!w) {
    np = 0;
    for (int i = threadIdx.x; i < half; i += 64, np++) {
      dxr[i] = f2bf(ga[np]);
      dxr[i + half] = f2bf(gb[np]);
    }
    return;
  }
  const bf16* xr = x + tok * ldx + h * D;
  float ss = 0.f, sxg = 0.f;
  np = 0;
  for (int i = threadIdx.x; i < half; i += 64, np++) {
    ga[np] = bf2f(f2bf(ga[np]));
    gb[np] = bf2f(f2bf(gb[np]));
    const float xa = bf2f(xr[i]), xb = bf2f(xr[i + half]);
    ss += xa * xa + xb * xb;
    sxg += xa * bf2f(w[i]) * ga[np] + xb * bf2f(w[i + half]) * gb[np];
  }
  ss = wave_sum(ss);
  sxg = wave_sum(sxg);
  const float r = rsqrtf(ss / (float)D + eps);
  const float coef = r * r * r * (sxg / (float)D);
  np = 0;
  for (int i = threadIdx.x; i < half; i += 64, np++) {
    const float xa = bf2f(xr[i]), xb = bf2f(xr[i + half]);
    dxr[i] = f2bf(r * bf2f(w[i]) * ga[np] - xa * coef);
    dxr[i + half] = f2bf(r * bf2f(w[i + half]) * gb[np] - xb * coef);
    atomicAdd(&dw[i], ga[np] * xa * r);
    atomicAdd(&dw[i + half], gb[np] * xb * r);
  }
}

// cos/sin of position * theta^(-2i/D), every intermediate in fp32 and in the reference's order
// of operations (precompute_freqs_cis, src/olmax/nn/rope.py:127-133): exponent = (2i)/D,
// freq = 1 / theta^exponent, angle = float(position) * freq.
__global__ __launch_bounds__(256) void rope_tables_kernel(float* __restrict__ cos_t, float* __restrict__ sin_t,
                                                          int seq_len, int half, float head_dim, float theta) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)seq_len * half) return;
  const int p = (int)(idx / half), i = (int)(idx % half);
  const float exponent = (float)(2 * i) / head_dim;
  const float freq = 1.0f / powf(theta, exponent);
  const float ang = (float)p * freq;
  cos_t[idx] = cosf(ang);
  sin_t[idx] = sinf(ang);
}

int grid_for(int64_t work_items, int per_block, int cap) {
  int64_t g = (work_items + per_block - 1) / per_block;
  if (g > cap) g = cap;
  if (g < 1) g = 1;
  return (int)g;
}

}  // namespace

// y = rms_norm(x, w) (+ res): res (optional, bf16 [rows, d]) is the residual stream added after
// the normalised value has been rounded to bf16 (post-norm layers: h = x + norm(f(x))).
extern "C" int32_t olmax_rmsnorm_fwd_res(hipStream_t stream, const void* x, const void* w,
                                         const void* res, void* y, int64_t rows, int32_t d,
                                         int64_t ldx, int64_t ldres, int64_t ldy, float eps) {
  if (rows == 0) return OLMAX_OK;
  OLMAX_CHECK(x && y, OLMAX_ERR_ARG, "olmax_rmsnorm_fwd: null pointer");
  OLMAX_CHECK(rows >= 0 && d > 0 && ldx >= d && ldy >= d && (!res || ldres >= d), OLMAX_ERR_SHAPE, "olmax_rmsnorm_fwd: bad shape rows=%ld d=%d", (long)rows, d);
  const bool vec = aligned16(x) && aligned16(y) && (!w || aligned16(w)) && ldx % 8 == 0 && ldy % 8 == 0 &&
                   (!res || (aligned16(res) && ldres % 8 == 0));
  const bf16 *xp = (const bf16*)x, *wp = (const bf16*)w, *rp = (const bf16*)res;
  bf16* yp = (bf16*)y;
  if (vec && d % 8 == 0 && d <= 256) {
    hipLaunchKernelGGL((rmsnorm_fwd_kernel<16, 2>), dim3(grid_for(rows, 16, 1 << 20)), dim3(256), 0, stream, xp, wp, rp, yp, rows, d, ldx, ldres, ldy, eps);
  } else if (vec && d % 8 == 0 && d <= 4096) {
    hipLaunchKernelGGL((rmsnorm_fwd_kernel<64, 8>), dim3(grid_for(rows, 4, 1 << 20)), dim3(256), 0, stream, xp, wp, rp, yp, rows, d, ldx, ldres, ldy, eps);
  } else if (vec && d % 8 == 0 && d <= 6144) {
    hipLaunchKernelGGL((rmsnorm_fwd_kernel<64, 12>), dim3(grid_for(rows, 4, 1 << 20)), dim3(256), 0, stream, xp, wp, rp, yp, rows, d, ldx, ldres, ldy, eps);
  } else if (vec && d % 8 == 0 && d <= 8192) {
    hipLaunchKernelGGL((rmsnorm_fwd_kernel<64, 16>), dim3(grid_for(rows, 4, 1 << 20)), dim3(256), 0, stream, xp, wp, rp, yp, rows, d, ldx, ldres, ldy, eps);
  } else {
    hipLaunchKernelGGL(rmsnorm_fwd_generic, dim3(grid_for(rows, 1, 1 << 16)), dim3(256), 0, stream, xp, wp, rp, yp, rows, d, ldx, ldres, ldy, eps);
  }
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}

extern "C" int32_t olmax_rmsnorm_fwd(hipStream_t stream, const void* x, const void* w, void* y,
                                     int64_t rows, int32_t d, int64_t ldx, int64_t ldy, float eps) {
  return olmax_rmsnorm_fwd_res(stream, x, w, nullptr, y, rows, d, ldx, 0, ldy, eps);
}

// dw (fp32, [d]) is ACCUMULATED into: the caller zeroes it.  dres (optional) is added to dx.
extern "C" int32_t olmax_rmsnorm_bwd(hipStream_t stream, const void* x, const void* w,
                                     const void* dy, const void* dres, void* dx, float* dw,
                                     int64_t rows, int32_t d, int64_t ldx, int64_t lddy,
                                     int64_t lddres, int64_t lddx, float eps) {
  if (rows == 0) return OLMAX_OK;
  OLMAX_CHECK(x && dy && dx, OLMAX_ERR_ARG, "olmax_rmsnorm_bwd: null pointer");
  OLMAX_CHECK(rows >= 0 && d > 0 && ldx >= d && lddy >= d && lddx >= d && (!dres || lddres >= d), OLMAX_ERR_SHAPE, "olmax_rmsnorm_bwd: bad shape");
  OLMAX_CHECK(!dw || w, OLMAX_ERR_ARG, "olmax_rmsnorm_bwd: dw requested without w");
  const bool vec = aligned16(x) && aligned16(dy) && aligned16(dx) && (!w || aligned16(w)) &&
                   (!dres || (aligned16(dres) && lddres % 8 == 0)) && ldx % 8 == 0 && lddy % 8 == 0 && lddx % 8 == 0;
  const bf16 *xp = (const bf16*)x, *wp = (const bf16*)w, *dyp = (const bf16*)dy, *drp = (const bf16*)dres;
  bf16* dxp = (bf16*)dx;
  const size_t smem = dw ? (size_t)d * 4 : 0;
#define OLMAX_NORM_BWD_ARGS smem, stream, xp, wp, dyp, drp, dxp, dw, rows, d, ldx, lddy, lddres, lddx, eps
  if (vec && d % 8 == 0 && d <= 256) {
    hipLaunchKernelGGL((rmsnorm_bwd_kernel<16, 2, 256>), dim3(grid_for(rows, 16, 256)), dim3(256), OLMAX_NORM_BWD_ARGS);
  } else if (vec && d % 8 == 0 && d <= 1024) {
    hipLaunchKernelGGL((rmsnorm_bwd_kernel<64, 2, 512>), dim3(grid_for(rows, 8, 256)), dim3(512), OLMAX_NORM_BWD_ARGS);
  } else if (vec && d % 8 == 0 && d <= 2048) {
    hipLaunchKernelGGL((rmsnorm_bwd_split_kernel<2, 2, 1024>), dim3(grid_for(rows, 8, 256)), dim3(1024), OLMAX_NORM_BWD_ARGS);
  } else if (vec && d % 8 == 0 && d <= 4096) {
    hipLaunchKernelGGL((rmsnorm_bwd_split_kernel<4, 2, 1024>), dim3(grid_for(rows, 4, 256)), dim3(1024), OLMAX_NORM_BWD_ARGS);
  } else if (vec && d % 8 == 0 && d <= 8192) {
    hipLaunchKernelGGL((rmsnorm_bwd_split_kernel<8, 2, 1024>), dim3(grid_for(rows, 2, 256)), dim3(1024), OLMAX_NORM_BWD_ARGS);
  } else {
    hipLaunchKernelGGL(rmsnorm_bwd_generic, dim3(grid_for(rows, 1, 1 << 16)), dim3(256), 0, stream, xp, wp, dyp, drp, dxp, dw, rows, d, ldx, lddy, lddres, lddx, eps);
  }
#undef OLMAX_NORM_BWD_ARGS
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}

// x,y: [tokens, heads*head_dim] views with row strides ldx/ldy (elements); in-place allowed.
// w != NULL fuses the head-wise RMSNorm (weight [head_dim]) in front of the rotation.
extern "C" int32_t olmax_qk_rope_fwd(hipStream_t stream, const void* x, void* y, const void* w,
                                     const float* cos_t, const float* sin_t, int64_t tokens,
                                     int32_t heads, int32_t head_dim, int32_t seq_len, int64_t ldx,
                                     int64_t ldy, float eps) {
  if (tokens == 0) return OLMAX_OK;
  OLMAX_CHECK(x && y && cos_t && sin_t, OLMAX_ERR_ARG, "olmax_qk_rope_fwd: null pointer");
  OLMAX_CHECK(tokens >= 0 && heads > 0 && head_dim > 0 && head_dim % 2 == 0 && seq_len > 0, OLMAX_ERR_SHAPE, "olmax_qk_rope_fwd: bad shape");
  OLMAX_CHECK(ldx >= (int64_t)heads * head_dim && ldy >= (int64_t)heads * head_dim, OLMAX_ERR_SHAPE, "olmax_qk_rope_fwd: row stride too small");
  const bf16* xp = (const bf16*)x;
  bf16* yp = (bf16*)y;
  if (head_dim == 128 && aligned16(x) && aligned16(y) && ldx % 8 == 0 && ldy % 8 == 0 && (!w || aligned16(w))) {
    const int64_t units = tokens * heads;
    dim3 grid((unsigned)((units + 15) / 16));
    if (w)
      hipLaunchKernelGGL(qk_rope_fwd_kernel<true>, grid, dim3(256), 0, stream, xp, yp, (const bf16*)w, cos_t, sin_t, tokens, heads, seq_len, ldx, ldy, eps);
    else
      hipLaunchKernelGGL(qk_rope_fwd_kernel<false>, grid, dim3(256), 0, stream, xp, yp, (const bf16*)nullptr, cos_t, sin_t, tokens, heads, seq_len, ldx, ldy, eps);
  } else {
    OLMAX_CHECK(head_dim <= 512, OLMAX_ERR_SHAPE, "olmax_qk_rope_fwd: head_dim > 512 unsupported");
    hipLaunchKernelGGL(qk_rope_fwd_generic, dim3((unsigned)(tokens * heads)), dim3(64), 0, stream, xp, yp, (const bf16*)w, cos_t, sin_t, tokens, heads, head_dim, seq_len, ldx, ldy, eps);
  }
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}

// dy: gradient w.r.t. the rotated (and normalised) q/k; dx: gradient w.r.t. the raw projection.
// With w: x is the raw projection saved from the forward, dw ([head_dim] fp32) is accumulated.
extern "C" int32_t olmax_qk_rope_bwd(hipStream_t stream, const void* dy, void* dx, const void* x,
                                     const void* w, float* dw, const float* cos_t,
                                     const float* sin_t, int64_t tokens, int32_t heads,
                                     int32_t head_dim, int32_t seq_len, int64_t lddy, int64_t lddx,
                                     int64_t ldx, float eps) {
  if (tokens == 0) return OLMAX_OK;
  OLMAX_CHECK(dy && dx && cos_t && sin_t, OLMAX_ERR_ARG, "olmax_qk_rope_bwd: null pointer");
  OLMAX_CHECK(!w || (x && dw), OLMAX_ERR_ARG, "olmax_qk_rope_bwd: norm fusion needs x and dw");
  OLMAX_CHECK(tokens >= 0 && heads > 0 && head_dim > 0 && head_dim % 2 == 0 && seq_len > 0, OLMAX_ERR_SHAPE, "olmax_qk_rope_bwd: bad shape");
  const bf16* dyp = (const bf16*)dy;
  bf16* dxp = (bf16*)dx;
  if (head_dim == 128 && aligned16(dy) && aligned16(dx) && lddy % 8 == 0 && lddx % 8 == 0 && (!w || (aligned16(w) && aligned16(x) && ldx % 8 == 0))) {
    const int64_t units = tokens * heads;
    dim3 grid((unsigned)((units + 15) / 16));
    if (w)
      hipLaunchKernelGGL(qk_rope_bwd_kernel<true>, dim3(grid.x < 1024 ? grid.x : 1024), dim3(256), 0, stream, dyp, dxp, (const bf16*)x, (const bf16*)w, dw, cos_t, sin_t, tokens, heads, seq_len, lddy, lddx, ldx, eps);
    else
      hipLaunchKernelGGL(qk_rope_bwd_kernel<false>, grid, dim3(256), 0, stream, dyp, dxp, (const bf16*)nullptr, (const bf16*)nullptr, (float*)nullptr, cos_t, sin_t, tokens, heads, seq_len, lddy, lddx, ldx, eps);
  } else {
    OLMAX_CHECK(head_dim <= 512, OLMAX_ERR_SHAPE, "olmax_qk_rope_bwd: head_dim > 512 unsupported");
    hipLaunchKernelGGL(qk_rope_bwd_generic, dim3((unsigned)(tokens * heads)), dim3(64), 0, stream, dyp, dxp, (const bf16*)x, (const bf16*)w, dw, cos_t, sin_t, tokens, heads, head_dim, seq_len, lddy, lddx, ldx, eps);
  }
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}

// cos/sin tables [seq_len, head_dim/2] fp32 for the rotary embedding, formed in fp32 as the
// reference forms them.
extern "C" int32_t olmax_rope_tables(hipStream_t stream, float* cos_t, float* sin_t, int32_t seq_len,
                                     int32_t head_dim, float theta) {
  OLMAX_CHECK(cos_t && sin_t, OLMAX_ERR_ARG, "olmax_rope_tables: null pointer");
  OLMAX_CHECK(seq_len > 0 && head_dim > 0 && head_dim % 2 == 0 && theta > 0.f, OLMAX_ERR_SHAPE, "olmax_rope_tables: bad shape or theta");
  const int half = head_dim / 2;
  const int64_t n = (int64_t)seq_len * half;
  hipLaunchKernelGGL(rope_tables_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, cos_t, sin_t, seq_len, half,
                     (float)head_dim, theta);
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}
