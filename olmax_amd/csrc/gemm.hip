// bf16 MFMA GEMM for gfx950 (MI355X): C[M,N] = A[M,K] * B[N,K]^T (+ R), fp32 accumulate.
//
// Replaces the cuBLASLt calls XLA issues for olmax.nn.functional.linear
// (reference src/olmax/nn/functional.py:14-27) and for the two transposed
// products its autodiff derives (dX = dY W, dW = dY^T X).
//
// One kernel template covers the three operand storage combinations:
//   A "KC": A[m*lda + k]   (reduction dim contiguous)   A "MC": A[k*lda + m]
//   B "KC": B[n*ldb + k]                                 B "NC": B[k*ldb + n]
// forward  Y = X W^T      : A=X  (KC), B=W  (KC)
// dX = dY W               : A=dY (KC), B=W  (NC)   (reduction over out-features)
// dW = dY^T X             : A=dY (MC), B=X  (NC)   (reduction over tokens)
//
// Tiling: BM x BN x 64 block tile, 64-lane waves each owning a WM x WN sub-tile as
// (WM/16) x (WN/16) v_mfma_f32_16x16x32_bf16 accumulators. Operand tiles stream from
// global memory straight into LDS (global_load_lds_dwordx4, no VGPR staging, no LDS-write
// phase) into the stage that is not being consumed; one barrier per k-tile. K-contiguous tiles live in LDS as [rows][64]; M/N-contiguous
// tiles live as [64][rows] and are read with ds_read_b64_tr_b16, the gfx950 transposing
// LDS load, which hands each lane 4 consecutive reduction-dim elements of its column.
//
// LDS bank geometry (measured on gfx950 with SQ_LDS_BANK_CONFLICT): 64 banks x 4 B, i.e.
// 256 B per clock.  ds_read_b128 serves 16 lanes per clock in the fixed groups
// {0-3,12-15,20-23,24-27}, {4-7,8-11,16-19,28-31} (+32 for the upper half); ds_read_b64
// serves lanes 0-31, then 32-63.  The 16-byte chunk index of every tile is XOR-swizzled so
// that each such group touches 16 distinct chunks modulo 256 B:
//   [rows][64]  (128 B rows, two rows per bank line): chunk ^= (row >> 1) & 7
//   [64][rows]  (a transposing read of 32 lanes covers k-rows {k..k+3} and {k+8..k+11},
//               32 B each): chunk ^= ((k & 3) << 2) | ((k >> 2) & 2)
//
// Workgroup -> tile mapping is XCD aware: hardware deals consecutive workgroup ids
// round-robin over the 8 XCDs, so id i is remapped to (i % 8) * (grid/8) + i / 8, giving
// every XCD one contiguous run of tiles; runs walk the tile grid in column groups so that
// the A row-panels and B column-panels a single L2 sees are re-used.
#include "common.h"
#include <atomic>
#include <mutex>
#include <type_traits>
#include <vector>

namespace {

constexpr int BK = 64;

#ifndef GEMM_VGPR_CAP
#define GEMM_VGPR_CAP
#endif

// Optional per-launch timing (HIP events recorded on the launch stream around every GEMM),
// switched on by olmax_gemm_profile_begin(); used by the benchmark's roofline report.
struct ProfRec {
  hipEvent_t e0, e1;
  double flops;
  double bytes;  // algorithmic: every operand and the result moved once
  int key;  // tile | a_kc<<12 | b_kc<<13 | has_res<<14 | out_f32<<15
  int M, N, K;
};
std::atomic<bool> g_prof_on{false};  // diagnostic switch, process-wide
std::vector<ProfRec> g_prof;
std::mutex g_prof_mu;

// GLU != 0 (1 silu, 2 tanh-gelu) turns the kernel into the fused gate/up projection of a gated
// MLP: B is [Wgate; Wup] ([2F, K]), a block covers 128 features and loads their 128 gate rows
// and 128 up rows, arranged in LDS so that every wave owns the gate AND the up columns of the
// same 32 features; the epilogue writes act = f(gate) * up ([M, F], leading dimension ldr) and,
// when Cv is given, gate|up ([M, 2F]) as the plain GEMM would.  N is F in that mode.
//
// EPI == 4 / 5 (silu / tanh-gelu) is the same projection run in the BACKWARD pass of a block whose
// forward kept nothing: gate and up are recomputed in the accumulators and, with the gradient of
// the activation output (dact [M, F], passed through the cos_t pointer with its row stride in
// seq_len), leave the kernel as act = f(gate) * up (R, for the down projection's weight gradient)
// and d gate | d up (Cv [M, 2F]) -- gate | up never reach memory and no separate GLU backward
// kernel runs.  Same roundings as olmax_gemm_glu_bf16 followed by olmax_glu_bwd.
//
// EPI == 3 is the fused q|k|v projection + rotary embedding: columns below rope_cols are heads of
// 128 that leave the kernel rotated (out = x cos + rotate_half(x) sin in fp32 on the bf16-rounded
// projection, as the separate RoPE kernel computes it); a wave's 64 columns are one half of a
// head and its neighbour (wave ^ 1) holds the other, so the rotation reads both from the LDS
// staging of the epilogue.  The position of a row is row % seq_len; cos/sin are [seq_len, 64] fp32.
template <int BM, int BN, int WM, int WN, bool A_KC, bool B_KC, bool HAS_RES, bool OUT_F32, int EPI = 0>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64) GEMM_VGPR_CAP void gemm_bf16_kernel(
    const bf16* __restrict__ A, const bf16* __restrict__ B, void* __restrict__ Cv,
    const bf16* __restrict__ R, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc,
    int64_t ldr, int tiles_m, int tiles_n, int c_vec, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int seq_len, int rope_cols, int order) {
  constexpr int GLU = (EPI == 1 || EPI == 2) ? EPI : (EPI == 4 ? 1 : (EPI == 5 ? 2 : 0));
  constexpr bool GLU_BWD = EPI == 4 || EPI == 5;
  constexpr bool ROPE = EPI == 3;
  static_assert(EPI == 0 || (BN == 256 && WN == 64 && B_KC && !HAS_RES && !OUT_F32), "fused epilogues: 256-wide NT tiles only");
  constexpr int NW = (BM / WM) * (BN / WN);
  constexpr int TM = WM / 16, TN = WN / 16;  // accumulators of 16x16 per wave
  constexpr int WAVES_N = BN / WN;
  constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2;
  constexpr int A_INS = A_BYTES / 1024 / NW;  // DMA instructions (1 KB each) per wave per k-tile
  constexpr int B_INS = B_BYTES / 1024 / NW;
  static_assert(A_INS >= 1 && B_INS >= 1, "tile too small for the wave count");
  constexpr int NINS = A_INS + B_INS;
  constexpr int STAGE = A_BYTES + B_BYTES;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];  // [A stage 0 | A stage 1 | B stage 0 | B stage 1]
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  // ---- XCD-aware tile assignment ----
  const int nwg = gridDim.x;
  int pid = blockIdx.x;
  int tile_m, tile_n;
  if (order > 0) {
    // Windows of 8 x 4 tiles (what the 32 CUs of an XCD hold at a time: 12 operand panels for
    // 32 tiles in that XCD's L2), dealt to the XCDs so that the 8 windows in flight together
    // form one block of `order` 8-row strips by 32 / order columns (order 2: 16 x 16 tiles, 32
    // distinct panels per round for the whole chip; order 4: 32 x 8; order 8: 64 x 4).  Groups of
    // `order` strips sweep all columns before the next group starts, so B is read once per group
    // and a group's A panels are re-read from the memory-side cache on every step of the sweep.
    // The tile grid is padded to whole windows and the launch to whole rounds; workgroups that
    // fall into the padding leave at once.
    const int xcd = pid & 7, slot = pid >> 3;
    const int c = (slot >> 5) * 8 + xcd, w = slot & 31;  // window, tile inside the window
    const int strips = (tiles_m + 7) >> 3, wpr = (tiles_n + 3) >> 2;  // 8-row strips, windows per strip
    if (c >= strips * wpr) return;
    const int full = (strips / order) * order * wpr;      // windows in whole groups of strips
    int sg, v, S;
    if (c < full) { sg = c / (order * wpr); v = c % (order * wpr); S = order; }
    else { sg = strips / order; v = c - full; S = strips % order; }
    tile_m = ((order * sg + v % S) << 3) + (w & 7);
    tile_n = ((v / S) << 2) + (w >> 3);
    if (tile_m >= tiles_m || tile_n >= tiles_n) return;
  } else {
    {
      const int per = nwg >> 3;
      if ((nwg & 7) == 0) pid = (pid & 7) * per + (pid >> 3);
    }
    // column-grouped walk: groups of GM row-tiles, sweep N inside a group
    constexpr int GM = 8;
    const int group_sz = GM * tiles_n;
    const int gid = pid / group_sz;
    const int first_m = gid * GM;
    const int gm = min(tiles_m - first_m, GM);
    tile_m = first_m + (pid % group_sz) % gm;
    tile_n = (pid % group_sz) / gm;
  }
  const int m0 = tile_m * BM, n0 = tile_n * (GLU ? BN / 2 : BN);  // GLU: first feature of the block

  // swizzles (see the bank-geometry note at the top of the file)
  auto kswz = [](int row) { return (row >> 1) & 7; };                         // [rows][64] tiles
  auto tswz = [](int kr) { return ((kr & 3) << 2) | ((kr >> 2) & 2); };        // [64][rows] tiles

  // ---- DMA sources: instruction i of this wave fills LDS block (i*NW + wave) of 1 KB, i.e.
  // 16-byte chunks p = block*64 + lane of the tile; the lane fetches whichever global chunk the
  // swizzle places there.  Consecutive instructions of a wave are a whole number of swizzle
  // periods (16 rows) apart, so a lane's byte offset inside the operand panel is one VGPR for all
  // of them; instruction and k-tile only move the wave-uniform base (SGPRs), and the loop spends
  // no vector instruction and one register per operand on DMA addresses.
  unsigned a_off, b_off;
  constexpr int A_IROWS = A_KC ? NW * 8 : NW * 64 / (BM / 8);  // tile rows between two instructions
  constexpr int B_IROWS = B_KC ? NW * 8 : NW * 64 / (BN / 8);
  static_assert(A_IROWS % 16 == 0 && B_IROWS % 16 == 0, "instructions of a wave must share the swizzle");
  static_assert(GLU == 0 || B_IROWS == 64, "GLU row mapping: one instruction per wave tile of 64 rows");
  {
    const int p = wave * 64 + lane;
    if (A_KC) {
      const int row = p >> 3, ph = p & 7;
      a_off = (unsigned)(((int64_t)row * lda + ((ph ^ kswz(row)) << 3)) * 2);
    } else {
      constexpr int CPR = BM / 8;  // chunks per k-row
      const int kr = p / CPR, ph = p % CPR;
      a_off = (unsigned)(((int64_t)kr * lda + ((ph ^ tswz(kr)) << 3)) * 2);
    }
    if (B_KC) {
      const int row = p >> 3, ph = p & 7;
      // GLU: LDS row (wave w: 64w .. 64w+63) = gate rows of features 32w .. 32w+31, then their up
      // rows; instruction i covers LDS rows 64i .. 64i+63, i.e. 32 features further on per step
      const int64_t grow = GLU ? (int64_t)((row >> 5) & 1) * N + (row & 31) : row;
      b_off = (unsigned)((grow * ldb + ((ph ^ kswz(row)) << 3)) * 2);
    } else {
      constexpr int CPR = BN / 8;
      const int kr = p / CPR, ph = p % CPR;
      b_off = (unsigned)(((int64_t)kr * ldb + ((ph ^ tswz(kr)) << 3)) * 2);
    }
  }
  const int64_t a_istep = (int64_t)A_IROWS * lda;  // elements between two instructions' sources
  const int64_t b_istep = (int64_t)(GLU ? 32 : B_IROWS) * ldb;
  const bf16* a_panel = A_KC ? A + (int64_t)m0 * lda : A + m0;  // k-tile 0 of this block's rows
  const bf16* b_panel = B_KC ? B + (int64_t)n0 * ldb : B + n0;
  const int64_t a_step = A_KC ? (int64_t)BK : (int64_t)BK * lda;
  const int64_t b_step = B_KC ? (int64_t)BK : (int64_t)BK * ldb;

  f32x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 4; r++) acc[i][j][r] = 0.f;

  const int KT = K / BK;
  const unsigned lds_base = lds_addr_of(smem);
  // issue DMA instructions [lo, hi) of the combined A+B list of k-tile kt into `stage`
  auto dma = [&](int kt, int stage, int lo, int hi) {
    const unsigned sa = lds_base + stage * A_BYTES;
    const unsigned sb = lds_base + 2 * A_BYTES + stage * B_BYTES;
#pragma unroll
    for (int i = 0; i < NINS; i++) {
      if (i < lo || i >= hi) continue;
      if (i < A_INS) {
        dma16_s(a_panel + (int64_t)kt * a_step + i * a_istep, a_off, sa + (i * NW + wave) * 1024);
      } else {
        const int j = i - A_INS;
        dma16_s(b_panel + (int64_t)kt * b_step + j * b_istep, b_off, sb + (j * NW + wave) * 1024);
      }
    }
  };

  // v_mfma_f32_16x16x32_bf16 operand geometry: lane -> row/column (lane % 16) of the 16-wide
  // tile, k-group lane / 16 (8 consecutive k each); accumulator lane -> column lane % 16,
  // rows 4*(lane/16) + r.  It sustains ~7 % more FLOP/s than the 32x32x16 form under the
  // board's power limit (less accumulator traffic per FLOP).
  const int l16 = lane & 15, g16 = lane >> 4;

  // Per-lane LDS byte addresses of the operand fragments, computed once.  LDS holds the A tiles
  // of both stages first, then the B tiles ([A0 | A1 | B0 | B1]), so that one base register
  // reaches a fragment of either stage with an immediate below 64 KB: for k-contiguous tiles one
  // base per k-step with stage and tile row (i*16 rows = i*2048 B) as immediate; for transposed
  // tiles one base per tile row -- the XOR swizzle permutes the chunk differently in every lane
  // -- with stage, k-step and half ((kk*32 + h*4) k-rows) as immediate.  The bases pass through
  // an empty asm so that the compiler keeps exactly these registers instead of re-deriving (and
  // spilling) one address per read; the loop then holds no address arithmetic at all.
  // (Adding whole 16-row tiles leaves kswz, which looks at row bits 1-3, unchanged; adding
  // multiples of 4 k-rows leaves tswz unchanged as long as bit 3 of the k-row comes from the
  // lane, which it does: k-row = 32*kk + 8*(lane/16) + 4*h + lane%16/4.)
  constexpr int NA_BASE = A_KC ? 2 : TM, NB_BASE = B_KC ? 2 : TN;
  static_assert(A_BYTES + 36 * (BM > BN ? BM : BN) * 2 < 65536, "fragment immediates must fit 16 bits");
  unsigned a_base[NA_BASE], b_base[NB_BASE];
#pragma unroll
  for (int x = 0; x < NA_BASE; x++) {
    unsigned v;
    if (A_KC) {  // x = k-step
      const int row = wm * WM + l16;
      v = row * 128 + (((x * 4 + g16) ^ kswz(row)) << 4);
    } else {     // x = tile row i
      const int col = wm * WM + x * 16 + ((l16 & 3) << 2);
      const int kr = g16 * 8 + (l16 >> 2);
      v = kr * (BM * 2) + (((col >> 3) ^ tswz(kr)) << 4) + ((col & 7) << 1);
    }
    v += lds_base;
    asm volatile("" : "+v"(v));
    a_base[x] = v;
  }
#pragma unroll
  for (int x = 0; x < NB_BASE; x++) {
    unsigned v;
    if (B_KC) {
      const int row = wn * WN + l16;
      v = row * 128 + (((x * 4 + g16) ^ kswz(row)) << 4);
    } else {
      const int col = wn * WN + x * 16 + ((l16 & 3) << 2);
      const int kr = g16 * 8 + (l16 >> 2);
      v = kr * (BN * 2) + (((col >> 3) ^ tswz(kr)) << 4) + ((col & 7) << 1);
    }
    v += lds_base + 2 * A_BYTES;
    asm volatile("" : "+v"(v));
    b_base[x] = v;
  }
  auto lds_b128 = [](unsigned addr) -> bf16x8 {
    return *reinterpret_cast<const __attribute__((address_space(3))) bf16x8*>((uintptr_t)addr);
  };
  auto lds_tr64 = [](unsigned addr) -> u32x2 {
    s16x4 t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(uintptr_t)addr);
    return (u32x2&)t;
  };
  // one operand fragment (16 rows x 32 k) of k-step kk (0 or 1) of stage st (all compile-time)
  auto load_a1 = [&](int st, int kk, int i) -> bf16x8 {
    if (A_KC) {
      return lds_b128(a_base[kk] + st * A_BYTES + i * 2048);
    } else {
      // transposing read: the 16-lane group g16 fetches k-rows kk*32 + 8*g16 + {0..3, 4..7}
      Pack8 p;
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const u32x2 t = lds_tr64(a_base[i] + st * A_BYTES + (kk * 32 + h * 4) * (BM * 2));
        p.u[h * 2 + 0] = t[0];
        p.u[h * 2 + 1] = t[1];
      }
      return p.v;
    }
  };
  auto load_b1 = [&](int st, int kk, int j) -> bf16x8 {
    if (B_KC) {
      return lds_b128(b_base[kk] + st * B_BYTES + j * 2048);
    } else {
      Pack8 p;
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const u32x2 t = lds_tr64(b_base[j] + st * B_BYTES + (kk * 32 + h * 4) * (BN * 2));
        p.u[h * 2 + 0] = t[0];
        p.u[h * 2 + 1] = t[1];
      }
      return p.v;
    }
  };

  // ---- main loop.  Software pipeline, all of it in registers and the two LDS stages:
  //   * fragments are double-buffered (fa/fb[0] = k-step 0, [1] = k-step 1 of a k-tile), and
  //     every LDS read is issued half a k-tile before the MFMAs that consume it;
  //   * the DMA of k-tile kt+2 goes into the stage k-tile kt occupied, right after the barrier
  //     that retires it, so it has a whole k-tile of MFMAs to land;
  //   * reads and DMA issues are slotted one per MFMA (pinned with sched_barrier), so that a
  //     wave never leaves the matrix pipe without work for longer than one MFMA;
  //   * the steady state has no branches: past the end the DMA re-fetches the last k-tile and
  //     the reads fetch a stage nobody uses any more.
  constexpr int NM = TM * TN, NF = TM + TN;
  // Register budget: B fragments are needed by every MFMA row of a half and are double-buffered;
  // an A fragment dies after its row (i-major MFMA order), so the first ASB of them are
  // single-buffered -- the next k-step's data is fetched into the same registers right behind the
  // row's last MFMA, a whole half ahead of its first use.  The last TM - ASB rows stay
  // double-buffered so that no fetch is issued within ~8 MFMAs of the barrier that waits for it.
  constexpr int ASB = BM == 256 ? 6 : 0, ND = TM - ASB;
  static_assert(2 * NINS <= NM && NF + 1 <= NM && NINS + NF <= NM, "not enough MFMA slots for the loads");
  static_assert(ASB == 0 || (NM >= 3 * NINS - 2 && NM >= 4 * (TN + ND)), "slot layout of the single-buffered scheme");
  bf16x8 fas[ASB > 0 ? ASB : 1], fad[2][ND], fb[2][TN];
  dma(0, 0, 0, NINS);
  if (KT > 1) {
    dma(1, 1, 0, NINS);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NINS) : "memory");  // k-tile 0 has landed
  } else {
    dma_wait_all();
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < TM; i++) {
    if (i < ASB) fas[i] = load_a1(0, 0, i);
    else fad[0][i - ASB] = load_a1(0, 0, i);
  }
#pragma unroll
  for (int j = 0; j < TN; j++) fb[0][j] = load_b1(0, 0, j);
  // running DMA bases: k-tile kt+2 while it exists, then they stop advancing
  const bf16* ap = a_panel + (int64_t)min(2, KT - 1) * a_step;
  const bf16* bp = b_panel + (int64_t)min(2, KT - 1) * b_step;
  // One k-tile.  The stage is a compile-time constant (the loop below is unrolled by two), so
  // every LDS address is a loop-invariant per-lane register plus an immediate: no address
  // arithmetic is left in the loop, where each vector instruction costs MFMA issue time.
  auto k_tile = [&](int kt, auto cur_tag) {
    constexpr int cur = decltype(cur_tag)::value;
    constexpr int nxt = cur ^ 1;
    const unsigned da = lds_base + cur * A_BYTES, db = lds_base + 2 * A_BYTES + cur * B_BYTES;
    // ---- first half: k-step 0 from registers; the fragments of k-step 1 are fetched meanwhile
    // (no fetch in slot 0: hoisted above the first MFMA it would make that MFMA's operand wait,
    // an in-order counter, cover the new read's latency as well)
#pragma unroll
    for (int m = 0; m < NM; m++) {
      const int i = m / TN, j = m % TN;
      acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[0][j], i < ASB ? fas[i] : fad[0][i < ASB ? 0 : i - ASB], acc[i][j], 0, 0, 0);
      if (m >= 1 && m <= TN) fb[1][m - 1] = load_b1(cur, 1, m - 1);
      if (m > TN && m <= TN + ND) fad[1][m - TN - 1] = load_a1(cur, 1, ASB + m - TN - 1);
      if (j == TN - 1 && i < ASB) fas[i] = load_a1(cur, 1, i);
      __builtin_amdgcn_sched_barrier(0);
    }
    // k-tile kt+1 has landed (issued one k-tile ago); every wave is done reading k-tile kt
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    // ---- second half: k-step 1 from registers; the slots issue the DMA of k-tile kt+2 into the
    // retired stage and fetch k-step 0 of k-tile kt+1; the first MFMA goes out right behind the barrier
#pragma unroll
    for (int m = 0; m < NM; m++) {
      const int i = m / TN, j = m % TN;
      acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[1][j], i < ASB ? fas[i] : fad[1][i < ASB ? 0 : i - ASB], acc[i][j], 0, 0, 0);
      int q = -1, f = -1;  // DMA instruction / double-buffered fragment of this slot
      if (ASB > 0) {
        // every third slot from 0: DMA (measured on the 7B step: issued on even slots from 2 the
        // step is 1.2 % slower, every 4th slot 0.6 %: the memory path likes an even request stream,
        // but the last DMA still needs most of a k-tile to land); slots 1, 5, 9, ...: B then
        // double-buffered A fragments
        if (m % 3 == 0 && m / 3 < NINS) q = m / 3;
        if ((m & 3) == 1 && (m >> 2) < TN + ND) f = m >> 2;
      } else {
        // DMA issues and fragment reads alternate while both last, from slot 1 when they fit
        constexpr int FIRST = (NINS + NF <= NM - 1) ? 1 : 0;
        constexpr int BOTH = NINS < NF ? NINS : NF;
        const int k = m - FIRST;
        if (k >= 0 && k < 2 * BOTH) { if (k & 1) f = k >> 1; else q = k >> 1; }
        else if (k >= 2 * BOTH && k < NINS + NF) { if (NINS > NF) q = k - BOTH; else f = k - BOTH; }
      }
      if (q >= 0) {
        if (q < A_INS) dma16_s(ap + q * a_istep, a_off, da + (q * NW + wave) * 1024);
        else dma16_s(bp + (q - A_INS) * b_istep, b_off, db + ((q - A_INS) * NW + wave) * 1024);
      }
      if (f >= 0) {
        if (f < TN) fb[0][f] = load_b1(nxt, 0, f);
        else fad[0][f - TN] = load_a1(nxt, 0, ASB + f - TN);
      }
      if (j == TN - 1 && i < ASB) fas[i] = load_a1(nxt, 0, i);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (kt + 3 < KT) {
      ap += a_step;
      bp += b_step;
    }
  };
  for (int kt = 0; kt + 1 < KT; kt += 2) {
    k_tile(kt, std::integral_constant<int, 0>());
    k_tile(kt + 1, std::integral_constant<int, 1>());
  }
  if (KT & 1) k_tile(KT - 1, std::integral_constant<int, 0>());
  dma_wait_all();  // the redundant tail DMAs must not outlive the workgroup's LDS allocation
  // The epilogue derives its addresses from a copy of the lane id that the compiler cannot see
  // through, so none of them is computed ahead of the loop and kept in registers across it.
  int lane_e = lane;
  asm volatile("" : "+v"(lane_e));
  const int l16e = lane_e & 15, g16e = lane_e >> 4;

  // ---- epilogue.  The MFMAs ran with their operands swapped (B fragment as the instruction's A),
  // so each accumulator is a transposed 16x16 tile: lane -> row l16e, columns 4*g16e + r, i.e. four
  // consecutive columns of one row of C per lane.
  if (GLU) {
    bf16* act = const_cast<bf16*>(R);
    bf16* gu = reinterpret_cast<bf16*>(Cv);
    if (c_vec == 2) {
      // Whole-line stores through LDS.  A wave's 128 x 32 features are half a line per row, so the
      // block's 256 x 128 output is staged wave by wave (64-byte rows, 16-byte chunks XOR-swizzled
      // by (row >> 2) & 3) and written out by rows: wave w takes rows 32w .. 32w+31, four rows of
      // 256 B per instruction.  First act, then (when kept for the backward pass) gate and up, or,
      // in the backward form, d gate and d up.
      constexpr int REG = WM * 64;  // bytes of one wave's staging region
      // backward form: this lane's gradients of the activation output, in accumulator layout
      // (8 bytes = its 4 features of one row), requested before the barrier that they ride out
      Pack4 dd[GLU_BWD ? TM : 1][2];
      if (GLU_BWD) {
        const bf16* dact = reinterpret_cast<const bf16*>(cos_t);
        const int64_t lddact = seq_len;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int j = 0; j < 2; j++)
            dd[i][j].u = *reinterpret_cast<const u32x2*>(dact + (int64_t)(m0 + wm * WM + i * 16 + l16e) * lddact + n0 + wn * 32 + j * 16 + g16e * 4);
      }
      __syncthreads();              // every wave is done reading the operand stages
#pragma unroll 1
      for (int pass = 0; pass < ((gu || GLU_BWD) ? 2 : 1); pass++) {
        if (pass) __syncthreads();  // the previous pass has been read back
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int j = 0; j < 2; j++) {
            const int row = i * 16 + l16e;
            unsigned char* dst = smem + wave * REG + row * 64 + ((((j << 1) | (g16e >> 1)) ^ ((row >> 2) & 3)) << 4) + ((g16e & 1) << 3);
            Pack4 pa, pg, pu;
#pragma unroll
            for (int r = 0; r < 4; r++) {
              // same roundings as the unfused path: gate and up are bf16 arrays, so is f(gate)
              pg.e[r] = f2bf(acc[i][j][r]);
              pu.e[r] = f2bf(acc[i][j + 2][r]);
              const float gf = bf2f(pg.e[r]);
              const float fg = GLU == 2 ? act_gelu(gf) : act_silu(gf);
              pa.e[r] = f2bf(bf2f(f2bf(fg)) * bf2f(pu.e[r]));
              if (GLU_BWD) {  // d gate = dact * up * f'(gate), d up = dact * f(gate)
                const float df = bf2f(dd[GLU_BWD ? i : 0][j].e[r]);
                pg.e[r] = f2bf(df * bf2f(pu.e[r]) * (GLU == 2 ? act_gelu_grad(gf) : act_silu_grad(gf)));
                pu.e[r] = f2bf(df * fg);
              }
            }
            if (pass == 0) {
              *reinterpret_cast<u32x2*>(dst) = pa.u;
            } else {
              *reinterpret_cast<u32x2*>(dst) = pg.u;
              *reinterpret_cast<u32x2*>(dst + 8 * REG) = pu.u;
            }
          }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < 8; t++) {
          const int row = wave * 32 + t * 4 + (lane_e >> 4), c = lane_e & 15;
          const int lrow = row & (WM - 1);
          const unsigned char* src = smem + ((row / WM) * WAVES_N + (c >> 2)) * REG + lrow * 64 + (((c & 3) ^ ((lrow >> 2) & 3)) << 4);
          if (pass == 0) {
            *reinterpret_cast<u32x4*>(act + (int64_t)(m0 + row) * ldr + n0 + c * 8) = *reinterpret_cast<const u32x4*>(src);
          } else {
            *reinterpret_cast<u32x4*>(gu + (int64_t)(m0 + row) * ldc + n0 + c * 8) = *reinterpret_cast<const u32x4*>(src);
            *reinterpret_cast<u32x4*>(gu + (int64_t)(m0 + row) * ldc + N + n0 + c * 8) = *reinterpret_cast<const u32x4*>(src + 8 * REG);
          }
        }
      }
      return;
    }
    if (GLU_BWD) return;  // the backward form is only launched with whole-line stores
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const int64_t row = m0 + wm * WM + i * 16 + l16e;
        const int col = n0 + wn * 32 + j * 16 + g16e * 4;  // first of this lane's 4 features
        Pack4 pa, pg, pu;
#pragma unroll
        for (int r = 0; r < 4; r++) {
          // same roundings as the unfused path: gate and up are bf16 arrays, so is f(gate)
          pg.e[r] = f2bf(acc[i][j][r]);
          pu.e[r] = f2bf(acc[i][j + 2][r]);
          const float gf = bf2f(pg.e[r]);
          const float a = bf2f(f2bf(GLU == 2 ? act_gelu(gf) : act_silu(gf)));
          pa.e[r] = f2bf(a * bf2f(pu.e[r]));
        }
        if (c_vec) {
          *reinterpret_cast<u32x2*>(act + row * ldr + col) = pa.u;
          if (gu) {
            *reinterpret_cast<u32x2*>(gu + row * ldc + col) = pg.u;
            *reinterpret_cast<u32x2*>(gu + row * ldc + N + col) = pu.u;
          }
        } else {
#pragma unroll
          for (int r = 0; r < 4; r++) {
            act[row * ldr + col + r] = pa.e[r];
            if (gu) {
              gu[row * ldc + col + r] = pg.e[r];
              gu[row * ldc + N + col + r] = pu.e[r];
            }
          }
        }
      }
    return;
  }
  if (!OUT_F32 && c_vec) {
    // Through LDS (free now), so that C leaves in whole 128-byte lines: each wave parks its
    // WM x 64 tile as bf16 rows of 128 B (16-byte chunks swizzled like the operand tiles), reads
    // it back 16 B per lane -- 8 lanes per row -- and stores 8 full lines per instruction.  A
    // residual joins on the way out, read in the same whole-line pattern: y = bf16(bf16(A B^T) + r),
    // the two roundings of the reference's `x + linear(...)` on bf16 arrays.
    static_assert(WN == 64, "the staging layout assumes 64-column wave tiles");
    __syncthreads();  // every wave is done reading the operand stages
    unsigned char* ws = smem + wave * (WM * 128);
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const int row = i * 16 + l16e;
        const int chunk = j * 2 + (g16e >> 1);
        Pack4 pk;
#pragma unroll
        for (int r = 0; r < 4; r++) pk.e[r] = f2bf(acc[i][j][r]);
        *reinterpret_cast<u32x2*>(ws + row * 128 + ((chunk ^ kswz(row)) << 4) + ((g16e & 1) << 3)) = pk.u;
      }
    bf16* C = reinterpret_cast<bf16*>(Cv);
    if (ROPE && n0 < rope_cols) {  // uniform over the block: rope_cols is a multiple of 256
      // Rotation on the way out.  Every wave has staged its half-heads; now wave w takes rows
      // 32w .. 32w+31 of the whole 256-column block, two rows (2 x 512 B) per instruction, so
      // that the four lanes of a row that need the same cos/sin entry (two heads x two halves)
      // sit in one instruction and share one request: the tables cost 128 KB per block, not 512.
      __syncthreads();
#pragma unroll 4
      for (int t = 0; t < 16; t++) {
        const int row = wave * 32 + t * 2 + (lane_e >> 5);      // row of the block
        const int c32 = lane_e & 31, chunk = c32 & 7;            // 16-byte chunk of the 512-byte row
        const int lrow = row & (WM - 1);                         // row inside the staging region
        const unsigned char* own = smem + ((row / WM) * WAVES_N + (c32 >> 3)) * (WM * 128) + lrow * 128 + ((chunk ^ kswz(lrow)) << 4);
        const unsigned char* oth = smem + ((row / WM) * WAVES_N + ((c32 >> 3) ^ 1)) * (WM * 128) + lrow * 128 + ((chunk ^ kswz(lrow)) << 4);
        Pack8 xo, xp, o;
        xo.u = *reinterpret_cast<const u32x4*>(own);
        xp.u = *reinterpret_cast<const u32x4*>(oth);
        const int pos = (m0 + row) % seq_len;
        const float* cp = cos_t + (int64_t)pos * 64 + chunk * 8;
        const float* sp = sin_t + (int64_t)pos * 64 + chunk * 8;
        const f32x4 c0 = *reinterpret_cast<const f32x4*>(cp), c1 = *reinterpret_cast<const f32x4*>(cp + 4);
        const f32x4 s0 = *reinterpret_cast<const f32x4*>(sp), s1 = *reinterpret_cast<const f32x4*>(sp + 4);
        const float sign = (c32 & 8) ? 1.f : -1.f;  // first half: x1 cos - x2 sin; second: x2 cos + x1 sin
#pragma unroll
        for (int e = 0; e < 8; e++) {
          const float cs = e < 4 ? c0[e & 3] : c1[e & 3], sn = e < 4 ? s0[e & 3] : s1[e & 3];
          o.e[e] = f2bf(bf2f(xo.e[e]) * cs + sign * bf2f(xp.e[e]) * sn);
        }
        *reinterpret_cast<u32x4*>(C + (int64_t)(m0 + row) * ldc + n0 + c32 * 8) = o.u;
      }
      return;
    }
    if (HAS_RES) {
      Pack8 rr[WM / 8];
#pragma unroll
      for (int t = 0; t < WM / 8; t++) {  // all residual lines requested before the first is needed
        const int row = t * 8 + (lane_e >> 3), chunk = lane_e & 7;
        rr[t].u = *reinterpret_cast<const u32x4*>(R + (int64_t)(m0 + wm * WM + row) * ldr + n0 + wn * WN + chunk * 8);
      }
#pragma unroll
      for (int t = 0; t < WM / 8; t++) {
        const int row = t * 8 + (lane_e >> 3), chunk = lane_e & 7;
        Pack8 line, o;
        line.u = *reinterpret_cast<const u32x4*>(ws + row * 128 + ((chunk ^ kswz(row)) << 4));
#pragma unroll
        for (int e = 0; e < 8; e++) o.e[e] = f2bf(bf2f(line.e[e]) + bf2f(rr[t].e[e]));
        *reinterpret_cast<u32x4*>(C + (int64_t)(m0 + wm * WM + row) * ldc + n0 + wn * WN + chunk * 8) = o.u;
      }
      return;
    }
#pragma unroll
    for (int t = 0; t < WM / 8; t++) {
      const int row = t * 8 + (lane_e >> 3), chunk = lane_e & 7;
      const u32x4 line = *reinterpret_cast<const u32x4*>(ws + row * 128 + ((chunk ^ kswz(row)) << 4));
      *reinterpret_cast<u32x4*>(C + (int64_t)(m0 + wm * WM + row) * ldc + n0 + wn * WN + chunk * 8) = line;
    }
    return;
  }
  // element-wise stores: fp32 output, or a C / R whose alignment rules out vector accesses
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const int64_t row = m0 + wm * WM + i * 16 + l16e;
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int col = n0 + wn * WN + j * 16 + g16e * 4 + r;
        float v = acc[i][j][r];
        if (HAS_RES) v = (OUT_F32 ? v : bf2f(f2bf(v))) + bf2f(R[row * ldr + col]);  // bf16 output: round, add, round
        if (OUT_F32)
          reinterpret_cast<float*>(Cv)[row * ldc + col] = v;
        else
          reinterpret_cast<bf16*>(Cv)[row * ldc + col] = f2bf(v);
      }
    }
}

// Bounds-checked scalar-FMA kernel for shapes the MFMA tiles do not divide
// (the reference's own unit tests use d_model=16, seq=12). One 16x16 output tile per block.
template <bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_generic_kernel(
    const bf16* __restrict__ A, const bf16* __restrict__ B, void* __restrict__ Cv,
    const bf16* __restrict__ R, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc,
    int64_t ldr, int a_kc, int b_kc) {
  __shared__ float As[16][17], Bs[16][17];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int row = blockIdx.y * 16 + ty, col = blockIdx.x * 16 + tx;
  float acc = 0.f;
  for (int k0 = 0; k0 < K; k0 += 16) {
    {
      const int m = blockIdx.y * 16 + ty, k = k0 + tx;
      As[ty][tx] = (m < M && k < K) ? bf2f(a_kc ? A[(int64_t)m * lda + k] : A[(int64_t)k * lda + m]) : 0.f;
      const int n = blockIdx.x * 16 + ty;
      Bs[ty][tx] = (n < N && k < K) ? bf2f(b_kc ? B[(int64_t)n * ldb + k] : B[(int64_t)k * ldb + n]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; k++) acc += As[ty][k] * Bs[tx][k];
    __syncthreads();
  }
  if (row < M && col < N) {
    if (R) acc = (OUT_F32 ? acc : bf2f(f2bf(acc))) + bf2f(R[(int64_t)row * ldr + col]);
    if (OUT_F32)
      reinterpret_cast<float*>(Cv)[(int64_t)row * ldc + col] = acc;
    else
      reinterpret_cast<bf16*>(Cv)[(int64_t)row * ldc + col] = f2bf(acc);
  }
}

std::atomic<int> g_order{0};  // diagnostic override of the tile order, process-wide: 0 automatic, -1 run order, > 0 that many strips
// How many 8-row strips of tiles the 8 XCDs' windows cover together (see the kernel), 0: the
// run order.  Measured inside the 7B train step (same box, alternating settings, per shape):
//   forward (both operands k-contiguous), weights that fit the memory-side cache: 1 strip
//     (all XCDs share the same 8 activation row panels and stream the weights): q|k|v -4.7 %;
//     a weight matrix beyond the cache (the LM head) wants every row in flight instead;
//   input gradients (dX = dY W): 2 strips, -2 % at K = 4096, -3.5 % on the LM head, else neutral;
//   weight gradients (dW = dY^T X): 4 strips, -3 % to -5 % on every shape.
// Grids that would need padded windows keep the run order (the padding costs more than it gains).
int tile_order(int tm, int tn, bool a_kc, bool b_kc, int N, int K) {
  const int o = g_order.load(std::memory_order_relaxed);
  if (o < 0) return 0;
  if (o > 0) return o;
  if (tm % 8 || tn % 4) return 0;
  const int strips = tm / 8;
  if (a_kc && b_kc) return (int64_t)N * K * 2 <= (128ll << 20) ? 1 : (strips < 8 ? strips : 8);
  if (a_kc) return strips < 2 ? strips : 2;
  return strips < 4 ? strips : 4;
}
unsigned order_grid(int order, int tm, int tn) {
  if (order <= 0) return (unsigned)(tm * tn);
  const int nwin = ((tm + 7) / 8) * ((tn + 3) / 4);
  return (unsigned)((nwin + 7) / 8 * 256);
}

template <int BM, int BN, int WM, int WN, bool A_KC, bool B_KC, bool HAS_RES, bool OUT_F32>
int launch_tile(hipStream_t s, const bf16* A, const bf16* B, void* C, const bf16* R, int M, int N,
                int K, int64_t lda, int64_t ldb, int64_t ldc, int64_t ldr) {
  constexpr int NT = (BM / WM) * (BN / WN) * 64;
  constexpr int SMEM = 2 * (BM + BN) * BK * 2;
  auto kern = gemm_bf16_kernel<BM, BN, WM, WN, A_KC, B_KC, HAS_RES, OUT_F32>;
  static std::once_flag attr_once;  // per instantiation
  std::call_once(attr_once, [&] { (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM); });
  const int tm = M / BM, tn = N / BN;
  ProfRec rec{};
  if (g_prof_on) {
    (void)hipEventCreate(&rec.e0);
    (void)hipEventCreate(&rec.e1);
    (void)hipEventRecord(rec.e0, s);
  }
  // vector epilogue: 16-byte stores to C, 16-byte loads from R
  const int c_vec = aligned16(C) && ldc % 8 == 0 && (!R || (aligned16(R) && ldr % 8 == 0));
  const int order = tile_order(tm, tn, A_KC, B_KC, N, K);
  hipLaunchKernelGGL(kern, dim3(order_grid(order, tm, tn)), dim3(NT), SMEM, s, A, B, C, R, M, N, K, lda, ldb, ldc,
                     ldr, tm, tn, c_vec, (const float*)nullptr, (const float*)nullptr, 1, 0, order);
  if (g_prof_on) {
    (void)hipEventRecord(rec.e1, s);
    rec.flops = 2.0 * M * N * K;
    rec.bytes = 2.0 * ((double)M * K + (double)N * K + (double)M * N * (HAS_RES ? 2 : 1) * (OUT_F32 ? 2 : 1));
    rec.key = (BM == 256 ? 256 : 128) | (A_KC << 12) | (B_KC << 13) | (HAS_RES << 14) | (OUT_F32 << 15);
    rec.M = M; rec.N = N; rec.K = K;
    std::lock_guard<std::mutex> lk(g_prof_mu);
    g_prof.push_back(rec);
  }
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}

// EPI 1 / 2: forward form (gu optional); 4 / 5: backward form (dact given, gu = d gate | d up)
template <int EPI>
int launch_glu(hipStream_t s, const bf16* A, const bf16* B, bf16* gu, bf16* act, int M, int F, int K, int64_t lda,
               int64_t ldb, int64_t ldgu, int64_t ldact, const bf16* dact = nullptr, int64_t lddact = 0) {
  constexpr int SMEM = 2 * (256 + 256) * BK * 2;
  auto kern = gemm_bf16_kernel<256, 256, 128, 64, true, true, false, false, EPI>;
  static std::once_flag attr_once;  // per instantiation
  std::call_once(attr_once, [&] { (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM); });
  const int tm = M / 256, tn = F / 128;
  ProfRec rec{};
  if (g_prof_on) {
    (void)hipEventCreate(&rec.e0);
    (void)hipEventCreate(&rec.e1);
    (void)hipEventRecord(rec.e0, s);
  }
  // 2: 16-byte stores of whole lines through LDS; 1: 8-byte stores straight from the accumulators
  const int c_vec = (aligned16(act) && ldact % 8 == 0 && (!gu || (aligned16(gu) && ldgu % 8 == 0 && F % 8 == 0))) ? 2
                    : ((((uintptr_t)act) & 7) == 0 && ldact % 4 == 0 && (!gu || ((((uintptr_t)gu) & 7) == 0 && ldgu % 4 == 0 && F % 4 == 0)));
  const int order = tile_order(tm, tn, true, true, 2 * F, K);
  hipLaunchKernelGGL(kern, dim3(order_grid(order, tm, tn)), dim3(512), SMEM, s, A, B, (void*)gu, (const bf16*)act, M, F, K, lda, ldb,
                     ldgu, ldact, tm, tn, c_vec, reinterpret_cast<const float*>(dact), (const float*)nullptr, (int)lddact, 0, order);
  if (g_prof_on) {
    (void)hipEventRecord(rec.e1, s);
    rec.flops = 4.0 * M * F * K;
    rec.bytes = 2.0 * ((double)M * K + 2.0 * F * K + (double)M * F * ((gu ? 3 : 1) + (dact ? 1 : 0)));
    rec.key = 256 | (1 << 12) | (1 << 13) | (1 << 16);
    rec.M = M; rec.N = 2 * F; rec.K = K;
    std::lock_guard<std::mutex> lk(g_prof_mu);
    g_prof.push_back(rec);
  }
  OLMAX_LAUNCH_CHECK();
  return OLMAX_OK;
}

template <bool A_KC, bool B_KC, bool HAS_RES, bool OUT_F32>
int dispatch_tile(hipStream_t s, const bf16* A, const bf16* B, void* C, const bf16* R, int M, int N,
                  int K, int64_t lda, int64_t ldb, int64_t ldc, int64_t ldr, int tile) {
  if (tile == 256)
    return launch_tile<256, 256, 128, 64, A_KC, B_KC, HAS_RES, OUT_F32>(s, A, B, C, R, M, N, K, lda,
                                                                        ldb, ldc, ldr);
  return launch_tile<128, 128, 64, 64, A_KC, B_KC, HAS_RES, OUT_F32>(s, A, B, C, R, M, N, K, lda,
                                                                     ldb, ldc, ldr);
}

std::atomic<int> g_force_tile{0};  // diagnostic override, process-wide

}  // namespace

extern "C" void olmax_gemm_set_tile(int tile) { g_force_tile = tile; }
extern "C" void olmax_gemm_set_order(int order) { g_order = order; }

// Start recording a HIP-event pair around every MFMA GEMM launch (diagnostic; allocates events).
extern "C" void olmax_gemm_profile_begin(void) {
  std::lock_guard<std::mutex> lk(g_prof_mu);
  g_prof.clear();
  g_prof_on = true;
}
// Stop recording, wait for the recorded events and aggregate per kernel instantiation.
// keys/ms/flops/launches: host arrays of `cap` entries; returns the number of distinct keys.
// key = tile | a_layout<<12 | b_layout<<13 | has_residual<<14 | out_f32<<15 | glu_epilogue<<16 | rope_epilogue<<17,
// with a_layout / b_layout bit SET when the operand is reduction-contiguous.  flops / bytes:
// algorithmic totals (2MNK; every operand and the result moved once).
extern "C" int32_t olmax_gemm_profile_end(int32_t* keys, double* ms, double* flops, double* bytes, int64_t* launches,
                                          int32_t cap) {
  std::lock_guard<std::mutex> lk(g_prof_mu);
  g_prof_on = false;
  int n = 0;
  for (auto& r : g_prof) {
    (void)hipEventSynchronize(r.e1);
    float t = 0.f;
    (void)hipEventElapsedTime(&t, r.e0, r.e1);
    int i = 0;
    for (; i < n; i++)
      if (keys[i] == r.key) break;
    if (i == n) {
      if (n >= cap) continue;
      keys[n] = r.key; ms[n] = 0; flops[n] = 0; bytes[n] = 0; launches[n] = 0;
      n++;
    }
    ms[i] += t; flops[i] += r.flops; bytes[i] += r.bytes; launches[i] += 1;
    (void)hipEventDestroy(r.e0);
    (void)hipEventDestroy(r.e1);
  }
  g_prof.clear();
  return n;
}

// As olmax_gemm_profile_end, aggregated per (key, M, N, K): mnk receives 3 ints per entry.
extern "C" int32_t olmax_gemm_profile_end_shapes(int32_t* keys, int32_t* mnk, double* ms, int64_t* launches, int32_t cap) {
  std::lock_guard<std::mutex> lk(g_prof_mu);
  g_prof_on = false;
  int n = 0;
  for (auto& r : g_prof) {
    (void)hipEventSynchronize(r.e1);
    float t = 0.f;
    (void)hipEventElapsedTime(&t, r.e0, r.e1);
    int i = 0;
    for (; i < n; i++)
      if (keys[i] == r.key && mnk[3 * i] == r.M && mnk[3 * i + 1] == r.N && mnk[3 * i + 2] == r.K) break;
    if (i == n) {
      if (n >= cap) continue;
      keys[n] = r.key; mnk[3 * n] = r.M; mnk[3 * n + 1] = r.N; mnk[3 * n + 2] = r.K; ms[n] = 0; launches[n] = 0;
      n++;
    }
    ms[i] += t; launches[i] += 1;
    (void)hipEventDestroy(r.e0);
    (void)hipEventDestroy(r.e1);
  }
  g_prof.clear();
  return n;
}

static int device_cu_count() {
  static std::atomic<int> n{0};  // every thread that finds 0 computes the same value
  int v = n.load(std::memory_order_relaxed);
  if (!v) {
    int dev = 0;
    if (!(hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)) v = 256;
    n.store(v, std::memory_order_relaxed);
  }
  return v;
}

extern "C" int32_t olmax_gemm_bf16(hipStream_t stream, const void* A, const void* B, void* C,
                                   const void* R, int32_t M, int32_t N, int32_t K, int64_t lda,
                                   int64_t ldb, int64_t ldc, int64_t ldr, int32_t a_layout,
                                   int32_t b_layout, int32_t out_f32) {
  OLMAX_CHECK(A && B && C, OLMAX_ERR_ARG, "olmax_gemm_bf16: null operand");
  OLMAX_CHECK(M > 0 && N > 0 && K > 0, OLMAX_ERR_SHAPE, "olmax_gemm_bf16: M,N,K must be positive (got %d,%d,%d)", M, N, K);
  OLMAX_CHECK((a_layout == 0 || a_layout == 1) && (b_layout == 0 || b_layout == 1), OLMAX_ERR_ARG,
              "olmax_gemm_bf16: layout flags must be 0 (reduction-contiguous) or 1");
  const bool a_kc = a_layout == 0, b_kc = b_layout == 0;
  OLMAX_CHECK(lda >= (a_kc ? K : M) && ldb >= (b_kc ? K : N) && ldc >= N && (!R || ldr >= N),
              OLMAX_ERR_SHAPE, "olmax_gemm_bf16: leading dimension smaller than row length");
  const bf16* a = (const bf16*)A;
  const bf16* b = (const bf16*)B;
  const bf16* r = (const bf16*)R;
  const bool vec_ok = aligned16(A) && aligned16(B) && (lda % 8 == 0) && (ldb % 8 == 0);
  int tile = 0;
  const int force_tile = g_force_tile.load(std::memory_order_relaxed);
  if (vec_ok && K % BK == 0) {
    if (M % 256 == 0 && N % 256 == 0 && (int64_t)(M / 256) * (N / 256) >= 128) tile = 256;
    else if (M % 128 == 0 && N % 128 == 0) tile = 128;
  }
  if (force_tile && tile) {
    if (force_tile == 256 && M % 256 == 0 && N % 256 == 0) tile = 256;
    if (force_tile == 128) tile = 128;
  }
  // Wave quantisation: with one 256x256 tile per CU per round, a last round that fills less
  // than half of the CUs (e.g. 1376 tiles = 5.375 rounds on 256 CUs) costs a whole round.
  // Such a problem is cut along M or N into a part whose tile count is a whole number of
  // rounds and a remainder that goes through this function again (and gets smaller tiles).
  if (tile == 256 && !force_tile) {
    const int ncu = device_cu_count();
    const int tm = M / 256, tn = N / 256;
    const int64_t tiles = (int64_t)tm * tn;
    const int rem = (int)(tiles % ncu);
    if (tiles > ncu && rem > 0 && rem * 2 < ncu) {
      int rm = 0, cn = 0;  // largest row-tile / column-tile counts giving whole rounds
      for (int x = tm - 1; x > 0; x--) if (((int64_t)x * tn) % ncu == 0) { rm = x; break; }
      for (int x = tn - 1; x > 0; x--) if (((int64_t)x * tm) % ncu == 0) { cn = x; break; }
      const size_t esz = out_f32 ? 4 : 2;
      if (rm > 0 && (int64_t)rm * tn >= (int64_t)cn * tm) {
        const int m1 = rm * 256;
        int rc = olmax_gemm_bf16(stream, A, B, C, R, m1, N, K, lda, ldb, ldc, ldr, a_layout, b_layout, out_f32);
        if (rc) return rc;
        const bf16* a2 = a_kc ? a + (int64_t)m1 * lda : a + m1;
        return olmax_gemm_bf16(stream, a2, B, (char*)C + (int64_t)m1 * ldc * esz, r ? r + (int64_t)m1 * ldr : nullptr,
                               M - m1, N, K, lda, ldb, ldc, ldr, a_layout, b_layout, out_f32);
      }
      if (cn > 0) {
        const int n1 = cn * 256;
        int rc = olmax_gemm_bf16(stream, A, B, C, R, M, n1, K, lda, ldb, ldc, ldr, a_layout, b_layout, out_f32);
        if (rc) return rc;
        const bf16* b2 = b_kc ? b + (int64_t)n1 * ldb : b + n1;
        return olmax_gemm_bf16(stream, A, b2, (char*)C + (int64_t)n1 * esz, r ? r + n1 : nullptr, M, N - n1, K, lda,
                               ldb, ldc, ldr, a_layout, b_layout, out_f32);
      }
    }
  }
  if (tile == 0) {
    dim3 grid((N + 15) / 16, (M + 15) / 16);
    if (out_f32)
      hipLaunchKernelGGL(gemm_generic_kernel<true>, grid, dim3(256), 0, stream, a, b, C, r, M, N, K,
                         lda, ldb, ldc, ldr, (int)a_kc, (int)b_kc);
    else
      hipLaunchKernelGGL(gemm_generic_kernel<false>, grid, dim3(256), 0, stream, a, b, C, r, M, N,
                         K, lda, ldb, ldc, ldr, (int)a_kc, (int)b_kc);
    OLMAX_LAUNCH_CHECK();
    return OLMAX_OK;
  }
#define GO(AK, BKC)                                                                              \
  do {                                                                                           \
    if (r) {                                                                                     \
      if (out_f32) return dispatch_tile<AK, BKC, true, true>(stream, a, b, C, r, M, N, K, lda, ldb, ldc, ldr, tile); \
      return dispatch_tile<AK, BKC, true, false>(stream, a, b, C, r, M, N, K, lda, ldb, ldc, ldr, tile);             \
    } else {                                                                                     \
      if (out_f32) return dispatch_tile<AK, BKC, false, true>(stream, a, b, C, r, M, N, K, lda, ldb, ldc, ldr, tile); \
      return dispatch_tile<AK, BKC, false, false>(stream, a, b, C, r, M, N, K, lda, ldb, ldc, ldr, tile);            \
    }                                                                                            \
  } while (0)
  if (a_kc && b_kc) GO(true, true);
  if (a_kc && !b_kc) GO(true, false);
  if (!a_kc && !b_kc) GO(false, false);
  GO(false, true);
#undef GO
}

extern "C" int32_t olmax_qk_rope_fwd(hipStream_t stream, const void* x, void* y, const void* w, const float* cos_t,
                                     const float* sin_t, int64_t tokens, int32_t heads, int32_t head_dim, int32_t seq_len,
                                     int64_t ldx, int64_t ldy, float eps);

// q|k|v projection with the rotary embedding of the q and k heads in the GEMM epilogue:
// out[M, N] = X W^T, then columns [0, rope_heads * 128) are rotated head by head (head_dim 128,
// position of row r = r % seq_len, cos/sin [seq_len, 64] fp32).  Equals olmax_gemm_bf16 followed
// by olmax_qk_rope_fwd in place on those columns, which is also what it falls back to when the
// shape does not fit the fused kernel.
extern "C" int32_t olmax_gemm_rope_bf16(hipStream_t stream, const void* X, const void* W, void* out, int32_t M, int32_t N,
                                        int32_t K, int64_t ldx, int64_t ldw, int64_t ldo, const float* cos_t,
                                        const float* sin_t, int32_t seq_len, int32_t rope_heads) {
  OLMAX_CHECK(X && W && out && cos_t && sin_t, OLMAX_ERR_ARG, "olmax_gemm_rope_bf16: null operand");
  OLMAX_CHECK(M > 0 && N > 0 && K > 0 && seq_len > 0 && rope_heads >= 0 && (int64_t)rope_heads * 128 <= N, OLMAX_ERR_SHAPE,
              "olmax_gemm_rope_bf16: bad shape (M %d N %d K %d seq_len %d rope_heads %d)", M, N, K, seq_len, rope_heads);
  OLMAX_CHECK(ldx >= K && ldw >= K && ldo >= N, OLMAX_ERR_SHAPE, "olmax_gemm_rope_bf16: leading dimension smaller than row length");
  const bool fits = aligned16(X) && aligned16(W) && aligned16(out) && aligned16(cos_t) && aligned16(sin_t) && ldx % 8 == 0 &&
                    ldw % 8 == 0 && ldo % 8 == 0 && K % BK == 0 && M % 256 == 0 && N % 256 == 0 && rope_heads % 2 == 0 &&
                    (int64_t)(M / 256) * (N / 256) >= 128 && !g_force_tile.load(std::memory_order_relaxed);
  if (fits) {
    constexpr int SMEM = 2 * (256 + 256) * BK * 2;
    auto kern = gemm_bf16_kernel<256, 256, 128, 64, true, true, false, false, 3>;
    static std::once_flag attr_once;  // per instantiation
    std::call_once(attr_once, [&] { (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM); });
    const int tm = M / 256, tn = N / 256;
    ProfRec rec{};
    if (g_prof_on) {
      (void)hipEventCreate(&rec.e0);
      (void)hipEventCreate(&rec.e1);
      (void)hipEventRecord(rec.e0, stream);
    }
    const int order = tile_order(tm, tn, true, true, N, K);
    hipLaunchKernelGGL(kern, dim3(order_grid(order, tm, tn)), dim3(512), SMEM, stream, (const bf16*)X, (const bf16*)W, out, (const bf16*)nullptr, M,
                       N, K, ldx, ldw, ldo, (int64_t)0, tm, tn, 1, cos_t, sin_t, seq_len, rope_heads * 128, order);
    if (g_prof_on) {
      (void)hipEventRecord(rec.e1, stream);
      rec.flops = 2.0 * M * N * K;
      rec.bytes = 2.0 * ((double)M * K + (double)N * K + (double)M * N);
      rec.key = 256 | (1 << 12) | (1 << 13) | (1 << 17);
      rec.M = M; rec.N = N; rec.K = K;
      std::lock_guard<std::mutex> lk(g_prof_mu);
      g_prof.push_back(rec);
    }
    OLMAX_LAUNCH_CHECK();
    return OLMAX_OK;
  }
  int rc = olmax_gemm_bf16(stream, X, W, out, nullptr, M, N, K, ldx, ldw, ldo, 0, 0, 0, 0);
  if (rc || rope_heads == 0) return rc;
  return olmax_qk_rope_fwd(stream, out, out, nullptr, cos_t, sin_t, M, rope_heads, 128, seq_len, ldo, ldo, 0.f);
}

extern "C" int32_t olmax_glu_fwd(hipStream_t stream, const void* gate, const void* up, void* out, int64_t T, int32_t F,
                                 int64_t ldg, int64_t ldu, int64_t ldo, int32_t act);

// Gated-MLP input projection with the activation fused into the GEMM epilogue:
// act_out[M, F] = f(X Wgate^T) * (X Wup^T), W = [Wgate; Wup] ([2F, K], row stride ldw); gu_out
// ([M, 2F], optional) receives gate|up for the backward pass.  Falls back to the plain GEMM
// plus olmax_glu_fwd (through a caller-provided gu_out) when the shape does not fit the tile.
extern "C" int32_t olmax_gemm_glu_bf16(hipStream_t stream, const void* X, const void* W, void* gu_out, void* act_out,
                                       int32_t M, int32_t F, int32_t K, int64_t ldx, int64_t ldw, int64_t ldgu,
                                       int64_t ldact, int32_t act) {
  OLMAX_CHECK(X && W && act_out, OLMAX_ERR_ARG, "olmax_gemm_glu_bf16: null operand");
  OLMAX_CHECK(M > 0 && F > 0 && K > 0, OLMAX_ERR_SHAPE, "olmax_gemm_glu_bf16: M,F,K must be positive (got %d,%d,%d)", M, F, K);
  OLMAX_CHECK(act == 0 || act == 1, OLMAX_ERR_ARG, "olmax_gemm_glu_bf16: act must be 0 (silu) or 1 (gelu-tanh)");
  OLMAX_CHECK(ldx >= K && ldw >= K && ldact >= F && (!gu_out || ldgu >= 2 * (int64_t)F), OLMAX_ERR_SHAPE,
              "olmax_gemm_glu_bf16: leading dimension smaller than row length");
  const bool fits = aligned16(X) && aligned16(W) && ldx % 8 == 0 && ldw % 8 == 0 && K % BK == 0 && M % 256 == 0 &&
                    F % 128 == 0 && (int64_t)(M / 256) * (F / 128) >= 128 && !g_force_tile.load(std::memory_order_relaxed);
  if (fits) {
    if (act == 0) return launch_glu<1>(stream, (const bf16*)X, (const bf16*)W, (bf16*)gu_out, (bf16*)act_out, M, F, K, ldx, ldw, ldgu, ldact);
    return launch_glu<2>(stream, (const bf16*)X, (const bf16*)W, (bf16*)gu_out, (bf16*)act_out, M, F, K, ldx, ldw, ldgu, ldact);
  }
  OLMAX_CHECK(gu_out, OLMAX_ERR_ARG, "olmax_gemm_glu_bf16: this shape needs gu_out as scratch for the unfused path");
  int rc = olmax_gemm_bf16(stream, X, W, gu_out, nullptr, M, 2 * F, K, ldx, ldw, ldgu, 0, 0, 0, 0);
  if (rc) return rc;
  return olmax_glu_fwd(stream, gu_out, (const bf16*)gu_out + F, act_out, M, F, ldgu, ldgu, ldact, act);
}

extern "C" int32_t olmax_glu_bwd(hipStream_t stream, const void* gate, const void* up, const void* dh, void* dgate, void* dup,
                                 int64_t T, int32_t F, int64_t ldg, int64_t ldu, int64_t lddh, int64_t lddg, int64_t lddu,
                                 int32_t act);

// The gated-MLP input projection re-run inside the backward pass (full-block recompute): from X, W = [Wgate; Wup] and
// dact = d loss / d (act(gate) * up) it produces act_out [M, F] (what the down projection's weight gradient needs) and
// dgu_out [M, 2F] = d gate | d up, without gate | up ever being written.  Equals olmax_gemm_glu_bf16 followed by
// olmax_glu_bwd, which is also the path taken (through dgu_out as scratch for gate | up) when the shape does not
// fit the tile.
extern "C" int32_t olmax_gemm_glu_bwd_bf16(hipStream_t stream, const void* X, const void* W, const void* dact, void* act_out,
                                           void* dgu_out, int32_t M, int32_t F, int32_t K, int64_t ldx, int64_t ldw,
                                           int64_t lddact, int64_t ldact, int64_t lddgu, int32_t act) {
  OLMAX_CHECK(X && W && dact && act_out && dgu_out, OLMAX_ERR_ARG, "olmax_gemm_glu_bwd_bf16: null operand");
  OLMAX_CHECK(M > 0 && F > 0 && K > 0, OLMAX_ERR_SHAPE, "olmax_gemm_glu_bwd_bf16: M,F,K must be positive (got %d,%d,%d)", M, F, K);
  OLMAX_CHECK(act == 0 || act == 1, OLMAX_ERR_ARG, "olmax_gemm_glu_bwd_bf16: act must be 0 (silu) or 1 (gelu-tanh)");
  OLMAX_CHECK(ldx >= K && ldw >= K && ldact >= F && lddact >= F && lddgu >= 2 * (int64_t)F, OLMAX_ERR_SHAPE,
              "olmax_gemm_glu_bwd_bf16: leading dimension smaller than row length");
  const bool fits = aligned16(X) && aligned16(W) && ldx % 8 == 0 && ldw % 8 == 0 && K % BK == 0 && M % 256 == 0 &&
                    F % 128 == 0 && (int64_t)(M / 256) * (F / 128) >= 128 && !g_force_tile.load(std::memory_order_relaxed) &&
                    aligned16(act_out) && ldact % 8 == 0 && aligned16(dgu_out) && lddgu % 8 == 0 &&
                    ((((uintptr_t)dact) & 7) == 0) && lddact % 4 == 0 && lddact < (1ll << 31);
  if (fits) {
    if (act == 0)
      return launch_glu<4>(stream, (const bf16*)X, (const bf16*)W, (bf16*)dgu_out, (bf16*)act_out, M, F, K, ldx, ldw, lddgu, ldact,
                           (const bf16*)dact, lddact);
    return launch_glu<5>(stream, (const bf16*)X, (const bf16*)W, (bf16*)dgu_out, (bf16*)act_out, M, F, K, ldx, ldw, lddgu, ldact,
                         (const bf16*)dact, lddact);
  }
  // unfused: gate | up into dgu_out, then the elementwise backward in place over it
  int rc = olmax_gemm_glu_bf16(stream, X, W, dgu_out, act_out, M, F, K, ldx, ldw, lddgu, ldact, act);
  if (rc) return rc;
  return olmax_glu_bwd(stream, dgu_out, (const bf16*)dgu_out + F, dact, dgu_out, (bf16*)dgu_out + F, M, F, lddgu, lddgu, lddact, lddgu,
                       lddgu, act);
}
