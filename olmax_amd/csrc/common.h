// Shared device/host helpers for the gfx950 kernels of libolmax_hip.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

typedef __bf16 bf16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define OLMAX_OK 0
#define OLMAX_ERR_ARG (-1)
#define OLMAX_ERR_SHAPE (-2)
#define OLMAX_ERR_ALIGN (-3)
#define OLMAX_ERR_LAUNCH (-4)
#define OLMAX_ERR_WORKSPACE (-5)

// Thread-local last error message (returned by olmax_last_error_string()).
int olmax_set_error(int code, const char* fmt, ...);

#define OLMAX_CHECK(cond, code, ...)                    \
  do {                                                  \
    if (!(cond)) return olmax_set_error(code, __VA_ARGS__); \
  } while (0)

#define OLMAX_LAUNCH_CHECK()                                                    \
  do {                                                                          \
    hipError_t e__ = hipGetLastError();                                         \
    if (e__ != hipSuccess)                                                      \
      return olmax_set_error(OLMAX_ERR_LAUNCH, "%s:%d launch failed: %s", __FILE__, __LINE__, \
                             hipGetErrorString(e__));                           \
  } while (0)

static inline bool aligned16(const void* p) { return (((uintptr_t)p) & 15) == 0; }

__device__ __forceinline__ float bf2f(bf16 x) { return (float)x; }
__device__ __forceinline__ bf16 f2bf(float x) { return (bf16)x; }

// 128-bit vector of 8 bf16, as raw words for loads/stores.
union Pack8 {
  u32x4 u;
  bf16x8 v;
  bf16 e[8];
};
union Pack4 {
  u32x2 u;
  bf16x4 v;
  bf16 e[4];
};

// 16 B per lane straight from global memory into LDS at (lds_addr + lane*16); lds_addr is
// wave-uniform (it travels in M0).  Issued as inline asm so that the compiler does not
// serialise later LDS reads behind it; the issuer waits for completion explicitly
// (s_waitcnt vmcnt) before the barrier that publishes the data.
__device__ __forceinline__ void dma16(const void* g, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(g) : "m0", "memory");
}
// Same, addressed as a wave-uniform 64-bit base (SGPR pair) plus a per-lane unsigned 32-bit
// byte offset: a lane's offset inside a tile is loop invariant, only the base moves.
__device__ __forceinline__ void dma16_s(const void* sbase, unsigned voff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "m0", "memory");
}
__device__ __forceinline__ void dma_wait_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
__device__ __forceinline__ unsigned lds_addr_of(const void* p) {
  return (unsigned)(uintptr_t)(__attribute__((address_space(3))) const unsigned char*)p;
}

// max / sum of a value with the one held by the lane 32 away (the other half of the wave),
// through v_permlane32_swap: no trip through the LDS crossbar (ds_bpermute) and its latency.
__device__ __forceinline__ float half_swap_max(float v) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_swap_sum(float v) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Wave64 all-reduce (sum) by xor shuffles.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Block-wide sum for blocks of NW waves; `red` is NW floats of LDS. All threads get the result.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  if (NW == 1) return v;
  const int w = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NW; i++) t += red[i];
  return t;
}
template <int NW>
__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  if (NW == 1) return v;
  const int w = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float t = red[0];
#pragma unroll
  for (int i = 1; i < NW; i++) t = fmaxf(t, red[i]);
  return t;
}

// api.hip: roctx ranges around phases of the whole-model entry points (no-ops unless switched on)
void olmax_range_push(const char* fmt, ...);
void olmax_range_pop(void);

// GLU activations (GatedMLP, reference src/olmax/nn/mlp.py:69-73): jax.nn.silu and the tanh
// form of jax.nn.gelu; shared by the elementwise GLU kernels and the GEMM's fused epilogue.
// silu(g) = g * sigmoid(g); the reciprocal is the hardware approximation (1 ulp), not the ~10-instruction
// IEEE division: the result is rounded to bf16 right away, and in the GEMM epilogue every
// vector instruction is time the matrix pipe idles.
__device__ __forceinline__ float act_silu(float g) { return g * __builtin_amdgcn_rcpf(1.f + __expf(-g)); }
// tanh(x) = 1 - 2 / (exp(2x) + 1): absolute error ~1e-7, saturates cleanly (exp -> inf gives 1,
// exp -> 0 gives -1); a handful of instructions where the library routine needs dozens of
// registers, which matters inside the GEMM epilogue.
__device__ __forceinline__ float fast_tanh(float x) {
  return 1.f - 2.f * __builtin_amdgcn_rcpf(__expf(2.f * x) + 1.f);
}
constexpr float GELU_C = 0.7978845608028654f;  // sqrt(2/pi)
__device__ __forceinline__ float act_gelu(float g) {
  return 0.5f * g * (1.f + fast_tanh(GELU_C * (g + 0.044715f * g * g * g)));
}

// derivatives of the two activations (the backward of act(gate) * up)
__device__ __forceinline__ float act_silu_grad(float g) {
  const float s = __builtin_amdgcn_rcpf(1.f + __expf(-g));  // as act_silu: hardware reciprocal, not a rounded division
  return s * (1.f + g * (1.f - s));
}
__device__ __forceinline__ float act_gelu_grad(float g) {
  const float t = fast_tanh(GELU_C * (g + 0.044715f * g * g * g));
  return 0.5f * (1.f + t) + 0.5f * g * (1.f - t * t) * GELU_C * (1.f + 3.f * 0.044715f * g * g);
}

// elementwise.hip, library-internal: olmax_adamw_dscale with the grid size (workgroups) exposed.
int olmax_adamw_grid(hipStream_t stream, float* p, const void* g, float* m, float* v, void* shadow_bf16, int64_t n,
                     int32_t grad_is_bf16, float lr, float b1, float b2, float eps, float wd, int64_t step,
                     float grad_scale, const float* grad_scale_dev, int grid_cap, const float* hyper_dev = nullptr);
