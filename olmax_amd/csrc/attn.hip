// Causal GQA flash attention for gfx950, head_dim 128, BSHD layout, bf16 in/out, fp32
// softmax statistics, optional sliding window and tanh logit soft-cap.
//
// Replaces the cuDNN fused-attention custom call that
// jax.nn.dot_product_attention(is_causal=True, local_window_size=w) lowers to
// (reference src/olmax/nn/attention.py:96-103) and its autodiff transpose.
// Mask: key j visible to query i iff j <= i and (w < 0 or j >= i - w).
//
// All three kernels keep the score tile TRANSPOSED in the MFMA accumulators so that each
// lane owns one query (forward, dQ) or one key (dK/dV) column: row statistics become
// per-lane scalars, and the exponentiated tile is already laid out as the B operand of the
// next v_mfma_f32_32x32x16_bf16 (k index = accumulator row pattern).  The operand that must
// be read against its storage order (V^T, K^T, Q^T, dO^T) comes from LDS through
// ds_read_b64_tr_b16.  K/V (or Q/dO) tiles are double buffered in LDS with a register-held
// prefetch of the next tile; 16-byte chunks are XOR-swizzled so that both ds_read_b128 and
// the transposing reads are bank-conflict free.
//
// Backward is split in two deterministic kernels (no atomics): dK/dV with the key tile
// stationary, dQ with the query tile stationary; each recomputes P from the saved LSE.
#include "common.h"
#include <mutex>
#include <type_traits>

extern "C" int32_t olmax_fill_zero(hipStream_t stream, void* p, int64_t nbytes);

namespace {

__device__ __forceinline__ float fexp2(float x) { return __builtin_amdgcn_exp2f(x); }
// tanh(raw * scale / cap) from a raw score, with c1 = 2 * scale * log2(e) / cap formed once per
// kernel: tanh(x) = 1 - 2 / (exp(2x) + 1) as one multiply, exp2, add, reciprocal and fma.  (Dividing
// by cap per score, as the formula reads, costs a correctly rounded division per element.)
__device__ __forceinline__ float cap_tanh(float raw, float c1) {
  return __builtin_fmaf(-2.f, __builtin_amdgcn_rcpf(fexp2(raw * c1) + 1.f), 1.f);
}

constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;

// 16-byte chunk swizzle of the [rows][128] tiles (256 B rows = one line of the 64 LDS banks).
// ds_read_b128 serves the lane groups {0-3,12-15,20-23,24-27} / {4-7,8-11,16-19,28-31} (one
// row per lane, same logical chunk) per clock and the transposing ds_read_b64 serves lanes
// 0-31 (4 consecutive rows x 4 chunks); this mask gives 16 distinct chunks in both cases.
__device__ __forceinline__ int swz(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }

// byte offset of 16B chunk `c` (0..15) of row `row` in a [rows][128] bf16 tile
__device__ __forceinline__ int tile_off(int row, int c) { return row * 256 + ((c ^ swz(row)) << 4); }

// Per-lane byte offsets of the operand fragments inside a [rows][128] tile.  The swizzle only
// looks at row bits 0-3, so stepping rows by 16 or 32 is a plain immediate offset and the
// eight (k-contiguous) plus eight (transposed) lane-dependent offsets are loop invariant.
// LEAN: the k-contiguous offsets are formed at each read from the first one (kc[s] = kc[0] ^ 32 s:
// the k-step only enters the XOR-swizzled chunk index) instead of living in eight registers, for a
// kernel that would otherwise spill them.
template <bool LEAN = false>
struct FragAddrT {
  int kc[LEAN ? 1 : 8];  // row (lane % 32), k-step s
  int tr[4][2];          // column tile dt, half h of the transposed read
  __device__ __forceinline__ void init(int lane) {
    const int l32 = lane & 31, lhi = lane >> 5;
#pragma unroll
    for (int s = 0; s < (LEAN ? 1 : 8); s++) kc[s] = l32 * 256 + (((2 * s + lhi) ^ swz(l32)) << 4);
    const int j16 = lane & 15, g16 = lane >> 4;
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const int col = dt * 32 + ((g16 & 1) << 4) + ((j16 & 3) << 2);
        const int row = ((g16 >> 1) << 2) + (h << 3) + (j16 >> 2);
        tr[dt][h] = row * 256 + (((col >> 3) ^ swz(row)) << 4) + ((col & 7) << 1);
      }
  }
  // k-contiguous fragment: rows row0 + lane%32 (row0 multiple of 16), k-step s
  __device__ __forceinline__ bf16x8 load_kc(const unsigned char* tile, int row0, int s) const {
    int off = kc[LEAN ? 0 : s];
    if (LEAN) {
      asm volatile("" : "+v"(off));  // keeps the XOR at the read: hoisted out of the loop it is a register again
      off ^= s << 5;
    }
    return *reinterpret_cast<const bf16x8*>(tile + off + row0 * 256);
  }
  // transposed fragment: MFMA rows = storage columns dt*32 + lane%32, k = storage rows r0 + {..}
  __device__ __forceinline__ bf16x8 load_tr(const unsigned char* tile, int r0, int dt) const {
    Pack8 p;
#pragma unroll
    for (int h = 0; h < 2; h++) {
      s16x4 t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(tile + tr[dt][h] + r0 * 256));
      p.u[h * 2 + 0] = ((u32x2&)t)[0];
      p.u[h * 2 + 1] = ((u32x2&)t)[1];
    }
    return p.v;
  }
};
typedef FragAddrT<false> FragAddr;

// A/B operand fragment with the k index contiguous in storage: row `row`, k-step s (16 wide)
__device__ __forceinline__ bf16x8 frag_kc(const unsigned char* tile, int row, int s, int lhi) {
  return *reinterpret_cast<const bf16x8*>(tile + tile_off(row, 2 * s + lhi));
}

// A operand fragment read transposed: rows of the MFMA = storage columns col0 + (lane % 32),
// k index = storage rows {r0 + 4*kg + 0..3, r0 + 8 + 4*kg + 0..3}
__device__ __forceinline__ bf16x8 frag_tr(const unsigned char* tile, int r0, int col0, int lane) {
  const int j16 = lane & 15, g16 = lane >> 4;
  const int col = col0 + ((g16 & 1) << 4) + ((j16 & 3) << 2);
  Pack8 p;
#pragma unroll
  for (int h = 0; h < 2; h++) {
    const int row = r0 + ((g16 >> 1) << 2) + (h << 3) + (j16 >> 2);
    const int off = row * 256 + ((((col >> 3)) ^ swz(row)) << 4) + ((col & 7) << 1);
    s16x4 t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(tile + off));
    p.u[h * 2 + 0] = ((u32x2&)t)[0];
    p.u[h * 2 + 1] = ((u32x2&)t)[1];
  }
  return p.v;
}

// Stream ROWS rows of 128 bf16 (global row r0 + i, clamped to S-1, row stride ld) into the
// swizzled LDS tile at lds_addr: ROWS/4 DMA instructions of 1 KB (4 rows) shared by 4 waves.
template <int ROWS>
__device__ __forceinline__ void dma_tile(const bf16* base, int64_t ld, int r0, int S, unsigned lds_addr, int wave, int lane) {
#pragma unroll
  for (int i = 0; i < ROWS / 16; i++) {
    const int blk = i * 4 + wave;
    const int p = blk * 64 + lane;
    const int row = p >> 4, ph = p & 15;
    const int gr = min(r0 + row, S - 1);
    dma16(base + (int64_t)gr * ld + ((ph ^ swz(row)) << 3), lds_addr + blk * 1024);
  }
}

// Workgroup id -> (tile rank, K/V group, head inside the group).  Hardware deals consecutive
// ids round-robin to the 8 XCDs and every XCD starts its ids in order, so the tile rank (the
// amount of causal work) is the SLOWEST index: each XCD gets the same mix of long and short
// tiles and starts the longest first (with the rank fastest, one XCD got 54 % more work than
// another and the CUs idled 39 % of the kernel).  When the group count divides by 8 the
// heads sharing a K/V head also land on one XCD, i.e. one L2.
struct WgCoord { int rank, group, r; };
__device__ __forceinline__ WgCoord decode_wg(int id, int ngroups, int rep) {
  const int level = ngroups * rep;
  WgCoord c;
  c.rank = id / level;
  const int u = id % level;
  if ((ngroups & 7) == 0) {
    const int blk = u / (8 * rep), rem = u % (8 * rep);
    c.r = rem >> 3;
    c.group = blk * 8 + (rem & 7);
  } else {
    c.group = u / rep;
    c.r = u % rep;
  }
  return c;
}

// The same tile transfer with everything lane-dependent hoisted out of the loop: a lane's byte
// offset (row * ld + swizzled chunk) inside a 16-row group is computed once, and since the
// swizzle only looks at row bits 0-3 the ROWS/16 DMA instructions of a transfer differ by a
// wave-uniform 16 * ld elements, which goes into the scalar base: one vector register per
// operand whatever the tile height.  Only for tiles that lie entirely inside the sequence (no
// row clamping).
template <int ROWS>
struct TileDma {
  unsigned off;
  int64_t step;
  __device__ __forceinline__ void init(int64_t ld, int wave, int lane) {
    const int p = wave * 64 + lane;
    const int row = p >> 4, ph = p & 15;
    off = (unsigned)((row * ld + ((ph ^ swz(row)) << 3)) * 2);
    step = 16 * ld;
  }
  __device__ __forceinline__ void issue(const bf16* row0, unsigned lds_addr, int wave) const {
#pragma unroll
    for (int i = 0; i < ROWS / 16; i++) dma16_s(row0 + i * step, off, lds_addr + (i * 4 + wave) * 1024);
  }
};

// acc + sum of the two bf16 values in dword w of a packed fragment
__device__ __forceinline__ float dot2_ones(const bf16x8& v, int w, float acc) {
  typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
  const bf2 pair = {v[2 * w], v[2 * w + 1]};
  const bf2 ones = {(__bf16)1.0f, (__bf16)1.0f};
  return __builtin_amdgcn_fdot2_f32_bf16(pair, ones, acc, false);
}

__device__ __forceinline__ bf16x8 pack_bf16x8(const f32x16& a, int base) {
  bf16x8 r;
#pragma unroll
  for (int e = 0; e < 8; e++) r[e] = f2bf(a[base + e]);
  return r;
}


// ---------------------------------------------------------------------------------------
// Forward.  grid = ceil(S/128)*H*B workgroups (see decode_wg); 256 threads; wave w owns queries i0+32w .. +31.
// ---------------------------------------------------------------------------------------
template <bool CAP>
__global__ __launch_bounds__(256, 2) void attn_fwd_kernel(
    const bf16* __restrict__ Q, const bf16* __restrict__ K, const bf16* __restrict__ V,
    bf16* __restrict__ O, float* __restrict__ LSE, int S, int H, int KH, int64_t ldq, int64_t ldk,
    int64_t ldv, int64_t ldo, float scale, int window, float cap) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];  // [2][K 16K | V 16K]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform for the compiler too
  const int l32 = lane & 31, lhi = lane >> 5;
  const int nqt = (S + 127) >> 7;
  const WgCoord wg = decode_wg(blockIdx.x, (int)(gridDim.x / (nqt * (H / KH))), H / KH);
  const int qt = nqt - 1 - wg.rank;  // longest rows first
  const int b = wg.group / KH, kh = wg.group % KH;
  const int h = kh * (H / KH) + wg.r;
  const int i0 = qt * 128;
  const int iw0 = i0 + wave * 32;  // first query of this wave
  const int qi = iw0 + l32;        // this lane's query
  const int qic = min(qi, S - 1);

  bf16x8 qf[8];
  {
    const bf16* qp = Q + ((int64_t)b * S + qic) * ldq + h * 128 + lhi * 8;
#pragma unroll
    for (int s = 0; s < 8; s++) qf[s] = *reinterpret_cast<const bf16x8*>(qp + s * 16);
  }
  const int j_lo = window >= 0 ? max(0, i0 - window) : 0;
  const int t_lo = j_lo >> 6;
  const int t_hi = min(i0 + 127, S - 1) >> 6;  // inclusive

  f32x16 o[4];
#pragma unroll
  for (int dt = 0; dt < 4; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[dt][r] = 0.f;
  float m = -INFINITY, lsum = 0.f;

  const bf16* kbase = K + (int64_t)b * S * ldk + kh * 128;
  const bf16* vbase = V + (int64_t)b * S * ldv + kh * 128;
  const unsigned lds0 = lds_addr_of(smem);
  const int wv = __builtin_amdgcn_readfirstlane(wave);
  TileDma<64> dk, dv;
  dk.init(ldk, wv, lane);
  dv.init(ldv, wv, lane);
  auto load_kv = [&](int t, int stage) {
    if (t * 64 + 64 <= S) {
      dk.issue(kbase + (int64_t)t * 64 * ldk, lds0 + stage * 32768, wv);
      dv.issue(vbase + (int64_t)t * 64 * ldv, lds0 + stage * 32768 + 16384, wv);
    } else {
      dma_tile<64>(kbase, ldk, t * 64, S, lds0 + stage * 32768, wv, lane);
      dma_tile<64>(vbase, ldv, t * 64, S, lds0 + stage * 32768 + 16384, wv, lane);
    }
  };
  const float sc2 = scale * LOG2E;
  const float cap_c1 = CAP ? 2.f * sc2 / cap : 0.f, cap_l2 = cap * LOG2E;  // soft-cap: see cap_tanh
  FragAddr fa;
  fa.init(lane);

  load_kv(t_lo, 0);
  dma_wait_all();
  __syncthreads();
  for (int t = t_lo; t <= t_hi; t++) {
    const int cur = (t - t_lo) & 1;
    if (t < t_hi) load_kv(t + 1, cur ^ 1);
    const int j0 = t * 64;
    // skip tiles this wave cannot see at all
    const bool visible = (j0 <= iw0 + 31) && (window < 0 || j0 + 63 >= iw0 - window);
    if (visible) {
      const unsigned char* sk = smem + cur * 32768;
      const unsigned char* sv = sk + 16384;
      f32x16 st[2];
#pragma unroll
      for (int jt = 0; jt < 2; jt++)
#pragma unroll
        for (int r = 0; r < 16; r++) st[jt][r] = 0.f;
#pragma unroll
      for (int s = 0; s < 8; s++)
#pragma unroll
        for (int jt = 0; jt < 2; jt++)
          st[jt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa.load_kc(sk, jt * 32, s), qf[s], st[jt], 0, 0, 0);
      // scores in log2 units
      if (CAP) {
#pragma unroll
        for (int jt = 0; jt < 2; jt++)
#pragma unroll
          for (int r = 0; r < 16; r++) st[jt][r] = cap_l2 * cap_tanh(st[jt][r], cap_c1);
      }
      const bool need_mask = (j0 + 63 > iw0) || (window >= 0 && j0 < iw0 + 31 - window);
      if (need_mask) {
#pragma unroll
        for (int jt = 0; jt < 2; jt++)
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int j = j0 + jt * 32 + (r >> 2) * 8 + lhi * 4 + (r & 3);
            const bool ok = (j <= qi) && (window < 0 || j >= qi - window);
            st[jt][r] = ok ? st[jt][r] : -INFINITY;
          }
      }
      float mt = -INFINITY;
#pragma unroll
      for (int jt = 0; jt < 2; jt++)
#pragma unroll
        for (int r = 0; r < 16; r++) mt = fmaxf(mt, st[jt][r]);
      if (!CAP) mt *= sc2;  // sc2 > 0: the max commutes with the scaling
      mt = half_swap_max(mt);
      // Lazy rescaling: the running reference m only moves when some row's maximum grew by more
      // than 2^8; until then exp2(s - m) <= 256 stays well inside fp32/bf16 range and the
      // 64-register rescale of O is skipped (wave-uniform decision).
      const bool grow = mt > m + 8.f;
      if (__builtin_amdgcn_ballot_w64(grow) != 0) {
        const float m_new = fmaxf(m, mt);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = fexp2(m - m_use);  // m = -inf -> 0
        lsum *= alpha;
        m = m_new;
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
#pragma unroll
          for (int r = 0; r < 16; r++) o[dt][r] *= alpha;
      }
      const float m_use = (m == -INFINITY) ? 0.f : m;
#pragma unroll
      for (int jt = 0; jt < 2; jt++)
#pragma unroll
        for (int r = 0; r < 16; r++)
          st[jt][r] = CAP ? fexp2(st[jt][r] - m_use) : fexp2(__builtin_fmaf(st[jt][r], sc2, -m_use));
      bf16x8 pb[4];
#pragma unroll
      for (int u = 0; u < 4; u++) pb[u] = pack_bf16x8(st[u >> 1], (u & 1) * 8);
      // row sum of the probabilities AS THE P.V PRODUCT SEES THEM (bf16), two per instruction
      // (v_dot2c_f32_bf16 against a pair of ones, two accumulators): numerator and denominator
      // of the softmax then carry the same rounding
      {
        float ps0 = 0.f, ps1 = 0.f;
#pragma unroll
        for (int u = 0; u < 4; u++) {
          ps0 = dot2_ones(pb[u], 0, ps0);
          ps1 = dot2_ones(pb[u], 1, ps1);
          ps0 = dot2_ones(pb[u], 2, ps0);
          ps1 = dot2_ones(pb[u], 3, ps1);
        }
        lsum += ps0 + ps1;
      }
#pragma unroll
      for (int u = 0; u < 4; u++)
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa.load_tr(sv, u * 16, dt), pb[u], o[dt], 0, 0, 0);
    }
    dma_wait_all();
    __syncthreads();
  }
  const float ltot = half_swap_sum(lsum);
  const float inv = ltot > 0.f ? 1.f / ltot : 0.f;
  if (qi < S) {
    bf16* op = O + ((int64_t)b * S + qi) * ldo + h * 128;
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        Pack4 pk;
#pragma unroll
        for (int e = 0; e < 4; e++) pk.e[e] = f2bf(o[dt][g * 4 + e] * inv);
        *reinterpret_cast<u32x2*>(op + dt * 32 + g * 8 + lhi * 4) = pk.u;
      }
    if (lhi == 0) LSE[((int64_t)b * H + h) * S + qi] = (m + log2f(ltot)) * LN2;
  }
}

// ---------------------------------------------------------------------------------------
// dQ.  Same tiling and grid as the forward; K/V tiles stream through LDS.
// ---------------------------------------------------------------------------------------
template <bool CAP>
__global__ __launch_bounds__(256, 2) void attn_bwd_dq_kernel(
    const bf16* __restrict__ Q, const bf16* __restrict__ K, const bf16* __restrict__ V,
    const bf16* __restrict__ O, const bf16* __restrict__ dO, const float* __restrict__ LSE,
    float* __restrict__ DELTA, bf16* __restrict__ dQ, int S, int H, int KH, int64_t ldq, int64_t ldk,
    int64_t ldv, int64_t ldo, int64_t lddo, int64_t lddq, float scale, int window, float cap) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform for the compiler too
  const int l32 = lane & 31, lhi = lane >> 5;
  const int nqt = (S + 127) >> 7;
  const WgCoord wg = decode_wg(blockIdx.x, (int)(gridDim.x / (nqt * (H / KH))), H / KH);
  const int qt = nqt - 1 - wg.rank;  // longest rows first
  const int b = wg.group / KH, kh = wg.group % KH;
  const int h = kh * (H / KH) + wg.r;
  const int i0 = qt * 128;
  const int iw0 = i0 + wave * 32;
  const int qi = iw0 + l32;
  const int qic = min(qi, S - 1);

  bf16x8 qf[8], dof[8];
  // delta[b,h,i] = sum_d dO[i,h,d] * O[i,h,d]: the two lanes of a query each hold half of its dO
  // row already, so the row sum costs one pass over O here; it is also written out for the dK/dV
  // kernel, which runs after this one.
  float dlt = 0.f;
  {
    const bf16* qp = Q + ((int64_t)b * S + qic) * ldq + h * 128 + lhi * 8;
    const bf16* dp = dO + ((int64_t)b * S + qic) * lddo + h * 128 + lhi * 8;
    const bf16* op = O + ((int64_t)b * S + qic) * ldo + h * 128 + lhi * 8;
#pragma unroll
    for (int s = 0; s < 8; s++) {
      qf[s] = *reinterpret_cast<const bf16x8*>(qp + s * 16);
      dof[s] = *reinterpret_cast<const bf16x8*>(dp + s * 16);
      const bf16x8 of = *reinterpret_cast<const bf16x8*>(op + s * 16);
#pragma unroll
      for (int e = 0; e < 8; e++) dlt += bf2f(of[e]) * bf2f(dof[s][e]);
    }
  }
  dlt = half_swap_sum(dlt);
  // stored NEGATED: the dK/dV kernel starts its dP accumulators from it, so that dP - delta
  // comes out of the MFMAs and costs that kernel no subtraction
  if (lhi == 0 && qi < S) DELTA[((int64_t)b * H + h) * S + qi] = -dlt;
  const float lse2 = LSE[((int64_t)b * H + h) * S + qic] * LOG2E;
  const int j_lo = window >= 0 ? max(0, i0 - window) : 0;
  const int t_lo = j_lo >> 6;
  const int t_hi = min(i0 + 127, S - 1) >> 6;

  f32x16 dq[4];
#pragma unroll
  for (int dt = 0; dt < 4; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) dq[dt][r] = 0.f;

  const bf16* kbase = K + (int64_t)b * S * ldk + kh * 128;
  const bf16* vbase = V + (int64_t)b * S * ldv + kh * 128;
  const unsigned lds0 = lds_addr_of(smem);
  const int wv = __builtin_amdgcn_readfirstlane(wave);
  TileDma<64> dk, dv;
  dk.init(ldk, wv, lane);
  dv.init(ldv, wv, lane);
  auto load_kv = [&](int t, int stage) {
    if (t * 64 + 64 <= S) {
      dk.issue(kbase + (int64_t)t * 64 * ldk, lds0 + stage * 32768, wv);
      dv.issue(vbase + (int64_t)t * 64 * ldv, lds0 + stage * 32768 + 16384, wv);
    } else {
      dma_tile<64>(kbase, ldk, t * 64, S, lds0 + stage * 32768, wv, lane);
      dma_tile<64>(vbase, ldv, t * 64, S, lds0 + stage * 32768 + 16384, wv, lane);
    }
  };
  const float sc2 = scale * LOG2E;
  const float cap_c1 = CAP ? 2.f * sc2 / cap : 0.f, cap_l2 = cap * LOG2E;  // soft-cap: see cap_tanh

  FragAddrT<CAP> fa;  // the soft-cap variant is the one short of registers
  fa.init(lane);

  load_kv(t_lo, 0);
  dma_wait_all();
  __syncthreads();
  for (int t = t_lo; t <= t_hi; t++) {
    const int cur = (t - t_lo) & 1;
    if (t < t_hi) load_kv(t + 1, cur ^ 1);
    const int j0 = t * 64;
    const bool visible = (j0 <= iw0 + 31) && (window < 0 || j0 + 63 >= iw0 - window);
    if (visible) {
      const unsigned char* sk = smem + cur * 32768;
      const unsigned char* sv = sk + 16384;
      const bool need_mask = (j0 + 63 > iw0) || (window >= 0 && j0 < iw0 + 31 - window);
      // dS of one 32-key half from its scores and dP, packed as the B operand of the dQ product
      bf16x8 dsb[4];
      auto finish_half = [&](int jt, f32x16& sj, const f32x16& dpj) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          float s = sj[r], chain = 1.f, p;
          if (CAP) {
            const float th = cap_tanh(s, cap_c1);
            p = fexp2(__builtin_fmaf(th, cap_l2, -lse2));
            chain = 1.f - th * th;
          } else {
            p = fexp2(__builtin_fmaf(s, sc2, -lse2));
          }
          if (need_mask) {
            const int j = j0 + jt * 32 + (r >> 2) * 8 + lhi * 4 + (r & 3);
            const bool ok = (j <= qi) && (window < 0 || j >= qi - window);
            p = ok ? p : 0.f;
          }
          sj[r] = p * (dpj[r] - dlt) * chain;
        }
        dsb[2 * jt] = pack_bf16x8(sj, 0);
        dsb[2 * jt + 1] = pack_bf16x8(sj, 8);
      };
      f32x16 st[2], dpt[2];
#pragma unroll
      for (int jt = 0; jt < 2; jt++) {
#pragma unroll
        for (int r = 0; r < 16; r++) { st[jt][r] = 0.f; dpt[jt][r] = 0.f; }
#pragma unroll
        for (int s = 0; s < 8; s++) {
          st[jt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa.load_kc(sk, jt * 32, s), qf[s], st[jt], 0, 0, 0);
          dpt[jt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa.load_kc(sv, jt * 32, s), dof[s], dpt[jt], 0, 0, 0);
        }
        // with the soft-cap's extra temporaries both halves do not fit the register file at once:
        // finish each half before the next one's products start
        if (CAP) finish_half(jt, st[jt], dpt[jt]);
      }
      if (!CAP) {
#pragma unroll
        for (int jt = 0; jt < 2; jt++) finish_half(jt, st[jt], dpt[jt]);
      }
#pragma unroll
      for (int u = 0; u < 4; u++)
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
          dq[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa.load_tr(sk, u * 16, dt), dsb[u], dq[dt], 0, 0, 0);
    }
    dma_wait_all();
    __syncthreads();
  }
  if (qi < S) {
    bf16* op = dQ + ((int64_t)b * S + qi) * lddq + h * 128;
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        Pack4 pk;
#pragma unroll
        for (int e = 0; e < 4; e++) pk.e[e] = f2bf(dq[dt][g * 4 + e] * scale);
        *reinterpret_cast<u32x2*>(op + dt * 32 + g * 8 + lhi * 4) = pk.u;
      }
  }
}

// ---------------------------------------------------------------------------------------
// dK/dV.  grid = ceil(S/128)*KH*B workgroups; wave w owns keys j0+32w..+31 (K and V fragments stay in
// registers); loops over the query heads of its group and over 32-row Q/dO tiles from the
// diagonal downwards.  LDS: 2 stages of (Q 8K | dO 8K | lse 128 B | delta 128 B) + V tile 32K.
// ---------------------------------------------------------------------------------------
template <bool CAP>
__global__ __launch_bounds__(256, 2) void attn_bwd_dkv_kernel(
    const bf16* __restrict__ Q, const bf16* __restrict__ K, const bf16* __restrict__ V,
    const bf16* __restrict__ dO, const float* __restrict__ LSE, const float* __restrict__ DELTA,
    bf16* __restrict__ dK, bf16* __restrict__ dV, int S, int H, int KH, int64_t ldq, int64_t ldk,
    int64_t ldv, int64_t lddo, int64_t lddk, int64_t lddv, float scale, int window, float cap) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int QT = 32;                   // query rows per iteration
  constexpr int STAGE = 2 * QT * 256 + 256;  // Q | dO | lse, delta
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform for the compiler too
  const int l32 = lane & 31, lhi = lane >> 5;
  // key tile 0 is seen by every query: rank order is already longest first
  const WgCoord wg = decode_wg(blockIdx.x, (int)(gridDim.x / ((S + 127) >> 7)), 1);
  const int kt = wg.rank;
  const int b = wg.group / KH, kh = wg.group % KH;
  const int rep = H / KH;
  const int j0 = kt * 128;
  const int jw0 = j0 + wave * 32;
  const int kj = jw0 + l32;  // this lane's key
  const int kjc = min(kj, S - 1);

  // K fragments of this wave's 32 keys stay in registers; the V tile of the whole workgroup
  // (128 keys) is parked in LDS behind the two stages and re-read as B operand every iteration
  bf16x8 kf[8];
  {
    const bf16* kp = K + ((int64_t)b * S + kjc) * ldk + kh * 128 + lhi * 8;
#pragma unroll
    for (int s = 0; s < 8; s++) kf[s] = *reinterpret_cast<const bf16x8*>(kp + s * 16);
  }
  f32x16 dk[4], dv[4];
#pragma unroll
  for (int dt = 0; dt < 4; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) { dk[dt][r] = 0.f; dv[dt][r] = 0.f; }

  const int i_hi = window >= 0 ? min(S - 1, j0 + 127 + window) : S - 1;
  const int t_lo = j0 / QT;
  const int t_hi = i_hi / QT;  // inclusive
  const int ntile = t_hi - t_lo + 1;
  const int total = ntile * rep;  // flattened (head, tile) iteration space
  const float sc2 = scale * LOG2E;
  const float cap_c1 = CAP ? 2.f * sc2 / cap : 0.f, cap_l2 = cap * LOG2E;  // soft-cap: see cap_tanh
  const unsigned lds0 = lds_addr_of(smem);
  const int wv = __builtin_amdgcn_readfirstlane(wave);

  float sreg = 0.f;
  TileDma<QT> tq, tdo;
  tq.init(ldq, wv, lane);
  tdo.init(lddo, wv, lane);
  // (head, tile) of the next tile to load; heads of the K/V group outermost
  int ld_h = kh * rep, ld_t = t_lo;
  auto load_tile = [&](int stage) {
    const int hq = ld_h, t = ld_t;
    if (++ld_t > t_hi) {
      ld_t = t_lo;
      ++ld_h;
    }
    if (t * QT + QT <= S) {
      tq.issue(Q + ((int64_t)b * S + t * QT) * ldq + hq * 128, lds0 + stage * STAGE, wv);
      tdo.issue(dO + ((int64_t)b * S + t * QT) * lddo + hq * 128, lds0 + stage * STAGE + QT * 256, wv);
    } else {
      dma_tile<QT>(Q + (int64_t)b * S * ldq + hq * 128, ldq, t * QT, S, lds0 + stage * STAGE, wv, lane);
      dma_tile<QT>(dO + (int64_t)b * S * lddo + hq * 128, lddo, t * QT, S, lds0 + stage * STAGE + QT * 256, wv, lane);
    }
    if (tid < 2 * QT) {
      const int ii = min(t * QT + (tid & (QT - 1)), S - 1);
      const float* src = tid < QT ? LSE : DELTA;
      sreg = src[((int64_t)b * H + hq) * S + ii];  // consumed by store_stats a whole iteration later
    }
  };
  // (the log2 scaling of LSE happens here, not at the load: touching the loaded value there
  // would make wave 0 wait out the memory latency at the top of every iteration)
  auto store_stats = [&](int stage) {
    if (tid < 2 * QT) reinterpret_cast<float*>(smem + stage * STAGE + 2 * QT * 256)[tid] = tid < QT ? sreg * LOG2E : sreg;
  };

  FragAddr fa;
  fa.init(lane);
  const unsigned char* svt = smem + 2 * STAGE;  // [128 keys][128] V tile
  dma_tile<128>(V + (int64_t)b * S * ldv + kh * 128, ldv, j0, S, lds0 + 2 * STAGE, wv, lane);
  load_tile(0);
  store_stats(0);
  dma_wait_all();
  __syncthreads();
  // One iteration on the tile in stage CUR (a compile-time constant, so that every LDS address
  // below is a loop-invariant register plus an immediate); `t` is the tile's query-tile index.
  auto iteration = [&](auto cur_tag, int t, bool more) {
    constexpr int CUR = decltype(cur_tag)::value;
    if (more) load_tile(CUR ^ 1);
    const int ib = t * QT;  // first query of the tile
    // this wave sees the tile iff some i in [ib, ib+QT) has j <= i <= j + window for its keys
    const bool visible = (ib + QT - 1 >= jw0) && (window < 0 || ib <= jw0 + 31 + window);
    if (visible) {
      const unsigned char* sq = smem + CUR * STAGE;
      const unsigned char* so = sq + QT * 256;
      const float* slse = reinterpret_cast<const float*>(sq + 2 * QT * 256);
      const float* sdel = slse + QT;
      // every (query, key) pair of the tile is visible unless the tile touches the diagonal, the
      // window edge or the end of the sequence
      const bool need_mask = (ib < jw0 + 31) || (ib + QT > S) || (window >= 0 && ib + QT - 1 > jw0 + window);
      f32x16 sa, dpa;
      // accumulator rows are queries i = ib + 8*(r/4) + 4*lhi + r%4; column = key kj.
      // dP starts from -delta of its query (what DELTA holds): the products then give dP - delta
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(sdel + g * 8 + lhi * 4);
#pragma unroll
        for (int e = 0; e < 4; e++) { sa[g * 4 + e] = 0.f; dpa[g * 4 + e] = d4[e]; }
      }
#pragma unroll
      for (int s = 0; s < 8; s++) {
        sa = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa.load_kc(sq, 0, s), kf[s], sa, 0, 0, 0);
        dpa = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa.load_kc(so, 0, s), fa.load_kc(svt, wave * 32, s), dpa, 0, 0, 0);
      }
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int il = g * 8 + lhi * 4;
        const f32x4 l4 = *reinterpret_cast<const f32x4*>(slse + il);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int r = g * 4 + e;
          const int i = ib + il + e;
          float s = sa[r], chain = 1.f, p;
          if (CAP) {
            const float th = cap_tanh(s, cap_c1);
            p = fexp2(__builtin_fmaf(th, cap_l2, -l4[e]));
            chain = 1.f - th * th;
          } else {
            p = fexp2(__builtin_fmaf(s, sc2, -l4[e]));
          }
          if (need_mask) {
            const bool ok = (kj <= i) && (i < S) && (window < 0 || kj >= i - window);
            p = ok ? p : 0.f;
          }
          sa[r] = p;
          dpa[r] = p * dpa[r] * chain;
        }
      }
      bf16x8 pb[2], dsb[2];
#pragma unroll
      for (int u = 0; u < 2; u++) {
        pb[u] = pack_bf16x8(sa, u * 8);
        dsb[u] = pack_bf16x8(dpa, u * 8);
      }
#pragma unroll
      for (int u = 0; u < 2; u++)
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
          dv[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa.load_tr(so, u * 16, dt), pb[u], dv[dt], 0, 0, 0);
          dk[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa.load_tr(sq, u * 16, dt), dsb[u], dk[dt], 0, 0, 0);
        }
    }
    if (more) store_stats(CUR ^ 1);
    dma_wait_all();
    __syncthreads();
  };
  {
    int t = t_lo;  // query tile being consumed
    for (int it = 0; it < total; it += 2) {
      iteration(std::integral_constant<int, 0>(), t, it + 1 < total);
      if (++t > t_hi) t = t_lo;
      if (it + 1 < total) {
        iteration(std::integral_constant<int, 1>(), t, it + 2 < total);
        if (++t > t_hi) t = t_lo;
      }
    }
  }
  if (kj < S) {
    bf16* kp = dK + ((int64_t)b * S + kj) * lddk + kh * 128;
    bf16* vp = dV + ((int64_t)b * S + kj) * lddv + kh * 128;
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        Pack4 pk, pv;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          pk.e[e] = f2bf(dk[dt][g * 4 + e] * scale);
          pv.e[e] = f2bf(dv[dt][g * 4 + e]);
        }
        *reinterpret_cast<u32x2*>(kp + dt * 32 + g * 8 + lhi * 4) = pk.u;
        *reinterpret_cast<u32x2*>(vp + dt * 32 + g * 8 + lhi * 4) = pv.u;
      }
  }
}

// ---------------------------------------------------------------------------------------
// Any head_dim (<= 256): one wave per (batch, head, query); scores staged in LDS.
// Used by the small shapes of unit tests and the CPU-sized reference configuration.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(64) void attn_fwd_generic(
    const bf16* __restrict__ Q, const bf16* __restrict__ K, const bf16* __restrict__ V,
    bf16* __restrict__ O, float* __restrict__ LSE, int S, int H, int KH, int D, int64_t ldq,
    int64_t ldk, int64_t ldv, int64_t ldo, float scale, int window, float cap) {
  extern __shared__ float sc[];  // S floats
  const int i = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int kh = h / (H / KH);
  const int lane = threadIdx.x;
  const bf16* q = Q + ((int64_t)b * S + i) * ldq + h * D;
  const int lo = window >= 0 ? max(0, i - window) : 0;
  float mx = -INFINITY;
  for (int j = lo + lane; j <= i; j += 64) {
    const bf16* k = K + ((int64_t)b * S + j) * ldk + kh * D;
    float s = 0.f;
    for (int d = 0; d < D; d++) s += bf2f(q[d]) * bf2f(k[d]);
    s *= scale;
    if (cap > 0.f) s = cap * tanhf(s / cap);
    sc[j] = s;
    mx = fmaxf(mx, s);
  }
  mx = wave_max(mx);
  float sm = 0.f;
  for (int j = lo + lane; j <= i; j += 64) sm += __expf(sc[j] - mx);
  sm = wave_sum(sm);
  const float lse = mx + __logf(sm);
  __syncthreads();
  for (int d = lane; d < D; d += 64) {
    float acc = 0.f;
    for (int j = lo; j <= i; j++) {
      const float p = bf2f(f2bf(__expf(sc[j] - lse)));
      acc += p * bf2f(V[((int64_t)b * S + j) * ldv + kh * D + d]);
    }
    O[((int64_t)b * S + i) * ldo + h * D + d] = f2bf(acc);
  }
  if (lane == 0) LSE[((int64_t)b * H + h) * S + i] = lse;
}

// dQ directly; dK/dV accumulated with fp32 atomics into [B*S, KH*D] workspaces.
__global__ __launch_bounds__(64) void attn_bwd_generic(
    const bf16* __restrict__ Q, const bf16* __restrict__ K, const bf16* __restrict__ V,
    const bf16* __restrict__ O, const bf16* __restrict__ dO, const float* __restrict__ LSE,
    bf16* __restrict__ dQ, float* __restrict__ dKf, float* __restrict__ dVf, int S, int H, int KH,
    int D, int64_t ldq, int64_t ldk, int64_t ldv, int64_t ldo, int64_t lddo, int64_t lddq,
    float scale, int window, float cap) {
  extern __shared__ float sh[];  // p[S], ds[S]
  float* sp = sh;
  float* sds = sh + S;
  const int i = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int kh = h / (H / KH);
  const int lane = threadIdx.x;
  const bf16* q = Q + ((int64_t)b * S + i) * ldq + h * D;
  const bf16* o = O + ((int64_t)b * S + i) * ldo + h * D;
  const bf16* go = dO + ((int64_t)b * S + i) * lddo + h * D;
  const float lse = LSE[((int64_t)b * H + h) * S + i];
  const int lo = window >= 0 ? max(0, i - window) : 0;
  float dl = 0.f;
  for (int d = lane; d < D; d += 64) dl += bf2f(o[d]) * bf2f(go[d]);
  dl = wave_sum(dl);
  for (int j = lo + lane; j <= i; j += 64) {
    const bf16* k = K + ((int64_t)b * S + j) * ldk + kh * D;
    const bf16* v = V + ((int64_t)b * S + j) * ldv + kh * D;
    float s = 0.f, dp = 0.f;
    for (int d = 0; d < D; d++) {
      s += bf2f(q[d]) * bf2f(k[d]);
      dp += bf2f(go[d]) * bf2f(v[d]);
    }
    s *= scale;
    float chain = 1.f;
    if (cap > 0.f) {
      const float th = tanhf(s / cap);
      s = cap * th;
      chain = 1.f - th * th;
    }
    const float p = __expf(s - lse);
    sp[j] = bf2f(f2bf(p));
    sds[j] = bf2f(f2bf(p * (dp - dl) * chain));
  }
  __syncthreads();
  for (int d = lane; d < D; d += 64) {
    float acc = 0.f;
    const float qd = bf2f(q[d]), god = bf2f(go[d]);
    for (int j = lo; j <= i; j++) {
      acc += sds[j] * bf2f(K[((int64_t)b * S + j) * ldk + kh * D + d]);
      atomicAdd(&dKf[((int64_t)b * S + j) * KH * D + kh * D + d], sds[j] * qd * scale);
      atomicAdd(&dVf[((int64_t)b * S + j) * KH * D + kh * D + d], sp[j] * god);
    }
    dQ[((int64_t)b * S + i) * lddq + h * D + d] = f2bf(acc * scale);
  }
}

__global__ void strided_cast_f32_bf16(const float* __restrict__ in, bf16* __restrict__ out,
                                      int64_t rows, int cols, int64_t ldo) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * cols) return;
  out[(i / cols) * ldo + i % cols] = f2bf(in[i]);
}

bool fast_ok(int D, const void* q, const void* k, const void* v, const void* o, int64_t ldq,
             int64_t ldk, int64_t ldv, int64_t ldo) {
  return D == 128 && aligned16(q) && aligned16(k) && aligned16(v) && aligned16(o) && ldq % 8 == 0 &&
         ldk % 8 == 0 && ldv % 8 == 0 && ldo % 8 == 0;
}

bool bwd_fast_ok(const void* q, const void* k, const void* v, const void* o, const void* d_o, const void* dq, const void* dk,
                 const void* dv, int D, int64_t ldq, int64_t ldk, int64_t ldv, int64_t ldo, int64_t lddo, int64_t lddq,
                 int64_t lddk, int64_t lddv) {
  return fast_ok(D, q, k, v, o, ldq, ldk, ldv, ldo) && aligned16(d_o) && aligned16(dq) && aligned16(dk) && aligned16(dv) &&
         lddo % 8 == 0 && lddq % 8 == 0 && lddk % 8 == 0 && lddv % 8 == 0;
}

constexpr int SM_KV = 2 * (2 * 32 * 256 + 256) + 128 * 256;
// dynamic-LDS limits of the backward kernels, set once per process
void bwd_fast_attributes() {
  static std::once_flag once;
  std::call_once(once, [] {
    (void)hipFuncSetAttribute((const void*)attn_bwd_dkv_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, SM_KV);
    (void)hipFuncSetAttribute((const void*)attn_bwd_dkv_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, SM_KV);
    (void)hipFuncSetAttribute((const void*)attn_bwd_dq_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
    (void)hipFuncSetAttribute((const void*)attn_bwd_dq_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
  });
}

// The two MFMA kernels of the backward pass (head_dim 128); delta: fp32 [B, H, S] scratch, fully
// written by the dQ kernel (each workgroup computes the entries of its own queries) before the
// dK/dV kernel, launched after it, reads them.
void launch_bwd_fast(hipStream_t stream, const bf16* qp, const bf16* kp, const bf16* vp, const bf16* op, const float* lse,
                     const bf16* gop, bf16* dq, bf16* dk, bf16* dv, float* delta, int B, int S, int H, int KH, int64_t ldq,
                     int64_t ldk, int64_t ldv, int64_t ldo, int64_t lddo, int64_t lddq, int64_t lddk, int64_t lddv, int window,
                     float softcap) {
  const float scale = 1.f / sqrtf(128.f);
  dim3 gkv((unsigned)(((S + 127) / 128) * KH * B)), gq((unsigned)(((S + 127) / 128) * H * B));
  bwd_fast_attributes();
  if (softcap > 0.f) {
    hipLaunchKernelGGL(attn_bwd_dq_kernel<true>, gq, dim3(256), 65536, stream, qp, kp, vp, op, gop, lse, delta, dq, S, H, KH, ldq, ldk, ldv, ldo, lddo, lddq, scale, window, softcap);
    hipLaunchKernelGGL(attn_bwd_dkv_kernel<true>, gkv, dim3(256), SM_KV, stream, qp, kp, vp, gop, lse, delta, dk, dv, S, H, KH, ldq, ldk, ldv, lddo, lddk, lddv, scale, window, softcap);
  } else {
    hipLaunchKernelGGL(attn_bwd_dq_kernel<false>, gq, dim3(256), 65536, stream, qp, kp, vp, op, gop, lse, delta, dq, S, H, KH, ldq, ldk, ldv, ldo, lddo, lddq, scale, window, softcap);
    hipLaunchKernelGGL(attn_bwd_dkv_kernel<false>, gkv, dim3(256), SM_KV, stream, qp, kp, vp, gop, lse, delta, dk, dv, S, H, KH, ldq, ldk, ldv, lddo, lddk, lddv, scale, window, softcap);
  }
}

}  // namespace

// q [B*S, ldq] (head h at columns h*D..), k/v [B*S, ldk/ldv] (KH heads), o [B*S, ldo],
// lse [B, H, S] fp32 (natural log of the masked softmax normaliser of the scaled, capped scores).
// window < 0: global causal; window >= 0: keys i-window..i.  softcap <= 0: off.
extern "C" int32_t olmax_attn_fwd(hipStream_t stream, const void* q, const void* k, const void* v,
                                  void* o, float* lse, int32_t B, int32_t S, int32_t H, int32_t KH,
                                  int32_t D, int64_t ldq, int64_t ldk, int64_t ldv, int64_t ldo,
                                  int32_t window, float softcap) {
  OLMAX_CHECK(q && k && v && o && lse, OLMAX_ERR_ARG, "olmax_attn_fwd: null pointer");
  OLMAX_CHECK(B > 0 && S > 0 && H > 0 && KH > 0 && D > 0 && H % KH == 0, OLMAX_ERR_SHAPE, "olmax_attn_fwd: bad shape B=%d S=%d H=%d KH=%d D=%d", B, S, H, KH, D);
  OLMAX_CHECK(ldq >= (int64_t)H * D && ldo >= (int64_t)H * D && ldk >= (int64_t)KH * D && ldv >= (int64_t)KH * D, OLMAX_ERR_SHAPE, "olmax_attn_fwd: row stride smaller than heads*head_dim");
  const float scale = 1.f / sqrtf((float)D);
  const bf16 *qp = (const bf16*)q, *kp = (const bf16*)k, *vp = (const bf16*)v;
  if (fast_ok(D, q, k, v, o, ldq, ldk, ldv, ldo)) {
    dim3 grid((unsigned)(((S + 127) / 128) * H * B));
    static std::once_flag once;
    std::call_once(once, [] {
      (void)hipFuncSetAttribute((const void*)attn_fwd_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
      (void)hipFuncSetAttribute((const void*)attn_fwd_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
    });
    if (softcap > 0.f) {
      hipLaunchKernelGGL(attn_fwd_kernel<true>, grid, dim3(256), 65536, stream, qp, kp, vp, (bf16*)o, lse, S, H, KH, ldq, ldk, ldv, ldo, scale, window, softcap);
    } else {
      hipLaunchKernelGGL(attn_fwd_kernel<false>, grid, dim3(256), 65536, stream, qp, kp, vp, (bf16*)o, lse, S, H, KH, ldq, ldk, ldv, ldo, scale, window, softcap);
    }
  } else {
    OLMAX_CHECK(D <= 256 && (size_t)S * 4 <= 65536, OLMAX_ERR_SHAPE, "olmax_attn_fwd: generic path supports head_dim <= 256 and seq_len <= 16384");
    hipLaunchKernelGGL(attn_fwd_generic, dim3(S, H, B), dim3(64), (size_t)S * 4, stream, qp, kp, vp, (bf16*)o, lse, S, H, KH, D, ldq, ldk, ldv, ldo, scale, window, softcap);
  }
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}

// Workspace: delta [B,H,S] fp32, then two fp32 [B*S, KH*D] accumulators for the generic path.
// Which path runs depends on head_dim AND on the alignment of the operands (a head_dim-128 call
// on unaligned views takes the generic path), which this query cannot see: it always returns the
// size that covers both.
static int64_t attn_delta_bytes(int32_t B, int32_t S, int32_t H) { return ((int64_t)B * H * S * 4 + 255) / 256 * 256; }
static int64_t attn_acc_bytes(int32_t B, int32_t S, int32_t KH, int32_t D) { return ((int64_t)B * S * KH * D * 4 + 255) / 256 * 256; }
extern "C" int64_t olmax_attn_bwd_workspace_bytes(int32_t B, int32_t S, int32_t H, int32_t KH, int32_t D) {
  return attn_delta_bytes(B, S, H) + 2 * attn_acc_bytes(B, S, KH, D);
}
// What the MFMA path alone needs (delta only): for callers that KNOW head_dim is 128 and every
// operand is 16-byte aligned with row strides that are multiples of 8.
extern "C" int64_t olmax_attn_bwd_workspace_bytes_aligned(int32_t B, int32_t S, int32_t H) { return attn_delta_bytes(B, S, H); }

extern "C" int32_t olmax_attn_bwd(hipStream_t stream, const void* q, const void* k, const void* v,
                                  const void* o, const float* lse, const void* d_o, void* dq, void* dk,
                                  void* dv, void* workspace, int64_t workspace_bytes, int32_t B,
                                  int32_t S, int32_t H, int32_t KH, int32_t D, int64_t ldq, int64_t ldk,
                                  int64_t ldv, int64_t ldo, int64_t lddo, int64_t lddq, int64_t lddk,
                                  int64_t lddv, int32_t window, float softcap) {
  OLMAX_CHECK(q && k && v && o && lse && d_o && dq && dk && dv && workspace, OLMAX_ERR_ARG, "olmax_attn_bwd: null pointer");
  OLMAX_CHECK(B > 0 && S > 0 && H > 0 && KH > 0 && D > 0 && H % KH == 0, OLMAX_ERR_SHAPE, "olmax_attn_bwd: bad shape");
  OLMAX_CHECK(workspace_bytes >= attn_delta_bytes(B, S, H) && (((uintptr_t)workspace) & 255) == 0, OLMAX_ERR_WORKSPACE, "olmax_attn_bwd: workspace too small or not 256-byte aligned");
  OLMAX_CHECK(ldq >= (int64_t)H * D && ldo >= (int64_t)H * D && lddo >= (int64_t)H * D && lddq >= (int64_t)H * D && ldk >= (int64_t)KH * D && ldv >= (int64_t)KH * D && lddk >= (int64_t)KH * D && lddv >= (int64_t)KH * D, OLMAX_ERR_SHAPE, "olmax_attn_bwd: row stride smaller than heads*head_dim");
  const float scale = 1.f / sqrtf((float)D);
  const bf16 *qp = (const bf16*)q, *kp = (const bf16*)k, *vp = (const bf16*)v, *op = (const bf16*)o, *gop = (const bf16*)d_o;
  float* delta = (float*)workspace;
  if (bwd_fast_ok(q, k, v, o, d_o, dq, dk, dv, D, ldq, ldk, ldv, ldo, lddo, lddq, lddk, lddv)) {
    launch_bwd_fast(stream, qp, kp, vp, op, lse, gop, (bf16*)dq, (bf16*)dk, (bf16*)dv, delta, B, S, H, KH, ldq, ldk, ldv, ldo, lddo,
                    lddq, lddk, lddv, window, softcap);
  } else {
    OLMAX_CHECK(D <= 256 && (size_t)S * 8 <= 65536, OLMAX_ERR_SHAPE, "olmax_attn_bwd: generic path supports head_dim <= 256 and seq_len <= 8192");
    const int64_t accb = attn_acc_bytes(B, S, KH, D);
    OLMAX_CHECK(workspace_bytes >= attn_delta_bytes(B, S, H) + 2 * accb, OLMAX_ERR_WORKSPACE,
                "olmax_attn_bwd: the generic path (head_dim != 128, or operands not 16-byte aligned) needs %ld workspace bytes",
                (long)(attn_delta_bytes(B, S, H) + 2 * accb));
    float* dkf = (float*)((char*)workspace + attn_delta_bytes(B, S, H));
    float* dvf = (float*)((char*)dkf + accb);
    { int rc = olmax_fill_zero(stream, dkf, 2 * accb); if (rc) return rc; }
    hipLaunchKernelGGL(attn_bwd_generic, dim3(S, H, B), dim3(64), (size_t)S * 8, stream, qp, kp, vp, op, gop, lse, (bf16*)dq, dkf, dvf, S, H, KH, D, ldq, ldk, ldv, ldo, lddo, lddq, scale, window, softcap);
    const int64_t n = (int64_t)B * S * KH * D;
    hipLaunchKernelGGL(strided_cast_f32_bf16, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, dkf, (bf16*)dk, (int64_t)B * S, KH * D, lddk);
    hipLaunchKernelGGL(strided_cast_f32_bf16, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, dvf, (bf16*)dv, (int64_t)B * S, KH * D, lddv);
  }
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}

// ---------------------------------------------------------------------------------------
// olmax_attn_bwd for callers that cannot allocate (code under HIP graph capture, serving loops,
// harnesses that forbid hipMalloc): the delta scratch lives in a file-scope device array
// instead of a caller-provided workspace.  Each GPU the library runs on holds its own copy of the
// array (4 MiB) until the process ends; every call on a GPU shares it, so calls that overlap on
// one GPU (two streams, two threads) race on it.  Nothing in it has to start at zero: the first
// kernel of a call writes every delta entry the second one reads.
// ---------------------------------------------------------------------------------------
constexpr int64_t ATTN_SCRATCH_FLOATS = 1 << 20;  // B * H * S <= 1 Mi (4 MiB)
static __device__ __align__(256) float scratch[ATTN_SCRATCH_FLOATS];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mu;
float* g_scratch_ptr[MAX_DEVICES];  // device address of `scratch` on each GPU, resolved on first use

// The array's name is only a host-side handle; its device address differs per GPU and comes
// from hipGetSymbolAddress with that GPU current.
// resolve == false: only look the address up (what a call under graph capture may do); the
// symbol query itself belongs to set-up, outside any capture.
int scratch_for_current_device(float** out, bool resolve) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES)
    return olmax_set_error(OLMAX_ERR_LAUNCH, "olmax_attn_bwd_noalloc: cannot identify the current device");
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    if (!resolve)
      return olmax_set_error(OLMAX_ERR_ARG,
                             "olmax_attn_bwd_noalloc: first use on this device is under stream capture; call "
                             "olmax_attn_bwd_noalloc_init() (or the entry point once, eagerly) before recording");
    float* p = nullptr;
    const hipError_t e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return olmax_set_error(OLMAX_ERR_LAUNCH, "olmax_attn_bwd_noalloc: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return OLMAX_OK;
}
}  // namespace

// Set-up for the current device: resolves the scratch address and sets the kernels' LDS limits.
// Call it once per device (with that device current) before recording olmax_attn_bwd_noalloc
// into a graph; an eager call of the entry point does the same.
extern "C" int32_t olmax_attn_bwd_noalloc_init(void) {
  float* p = nullptr;
  bwd_fast_attributes();
  return scratch_for_current_device(&p, true);
}

extern "C" int64_t olmax_attn_bwd_noalloc_max_rows(void) { return ATTN_SCRATCH_FLOATS; }

extern "C" int32_t olmax_attn_bwd_noalloc(hipStream_t stream, const void* q, const void* k, const void* v,
                                          const void* o, const float* lse, const void* d_o, void* dq, void* dk,
                                          void* dv, int32_t B, int32_t S, int32_t H, int32_t KH, int32_t D,
                                          int64_t ldq, int64_t ldk, int64_t ldv, int64_t ldo, int64_t lddo,
                                          int64_t lddq, int64_t lddk, int64_t lddv, int32_t window, float softcap) {
  OLMAX_CHECK(q && k && v && o && lse && d_o && dq && dk && dv, OLMAX_ERR_ARG, "olmax_attn_bwd_noalloc: null pointer");
  OLMAX_CHECK(B > 0 && S > 0 && H > 0 && KH > 0 && D > 0 && H % KH == 0, OLMAX_ERR_SHAPE, "olmax_attn_bwd_noalloc: bad shape");
  OLMAX_CHECK(ldq >= (int64_t)H * D && ldo >= (int64_t)H * D && lddo >= (int64_t)H * D && lddq >= (int64_t)H * D && ldk >= (int64_t)KH * D && ldv >= (int64_t)KH * D && lddk >= (int64_t)KH * D && lddv >= (int64_t)KH * D, OLMAX_ERR_SHAPE, "olmax_attn_bwd_noalloc: row stride smaller than heads*head_dim");
  OLMAX_CHECK((int64_t)B * H * S <= ATTN_SCRATCH_FLOATS, OLMAX_ERR_WORKSPACE,
              "olmax_attn_bwd_noalloc: batch*heads*seq_len = %ld exceeds the built-in scratch of %ld rows; use olmax_attn_bwd with a workspace",
              (long)((int64_t)B * H * S), (long)ATTN_SCRATCH_FLOATS);
  OLMAX_CHECK(bwd_fast_ok(q, k, v, o, d_o, dq, dk, dv, D, ldq, ldk, ldv, ldo, lddo, lddq, lddk, lddv), OLMAX_ERR_ALIGN,
              "olmax_attn_bwd_noalloc: needs head_dim 128, 16-byte aligned pointers and row strides that are multiples of 8; use olmax_attn_bwd otherwise");
  float* delta = nullptr;
  {
    // under capture only a pointer resolved earlier may be used: the symbol query is set-up work
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    const bool capturing = stream && hipStreamIsCapturing(stream, &st) == hipSuccess && st == hipStreamCaptureStatusActive;
    int rc = scratch_for_current_device(&delta, !capturing);
    if (rc) return rc;
  }
  launch_bwd_fast(stream, (const bf16*)q, (const bf16*)k, (const bf16*)v, (const bf16*)o, lse, (const bf16*)d_o, (bf16*)dq, (bf16*)dk,
                  (bf16*)dv, delta, B, S, H, KH, ldq, ldk, ldv, ldo, lddo, lddq, lddk, lddv, window, softcap);
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}
