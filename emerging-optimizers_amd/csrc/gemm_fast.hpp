// Fast path of the bf16 tile engine for the MFMA-bound shapes (K % 64 == 0, no K tail; row edges are
// allowed and handled by clamped loads plus a guarded epilogue).
//
// A variant is described by FastCfg: square workgroup tile, wavefront grid, ring-slot depth BK and number
// of ring slots.  Global -> LDS goes through the direct-to-LDS load (16 bytes per lane, a wavefront fills
// 1 KB of LDS at base + 16 * lane); the slots form a ring with one barrier per K tile (see the kernel).
// Because LDS placement is fixed by the lane id, swizzling is done by choosing which global chunk a
// lane fetches:
//   K-contiguous operand: LDS row = 128 B (8 chunks); chunk c of row r sits at slot c ^ ((r >> 1) & 7),
//     so the 16 rows one quarter-wave reads with ds_read_b128 cover all 64 banks.
//   K-strided operand: LDS row = one k (256 values = 32 chunks); chunk c of row k sits at slot
//     (c + 4 k) mod 32; fragments are fetched with the LDS transpose read ds_read_b64_tr_b16, which
//     returns to lane i of a 16-lane group the four k-values of column i from four consecutive k-rows.
#pragma once
#include "gemm_engine.hpp"

namespace mi {

typedef short s16x4_t __attribute__((ext_vector_type(4)));

// Compile-time shape of one fast-kernel variant.
template <int TILE_M_, int WGM_, int WGN_, int BK_, int NS_, int KSPLIT_ = 1, int TILE_N_ = TILE_M_>
struct FastCfg {
  static constexpr int TILE_M = TILE_M_, TILE_N = TILE_N_;  // workgroup tile: rows of P x rows of Q
  static constexpr int TILE = TILE_M_;                      // (SYRK uses square tiles)
  // KSPLIT groups of WGM x WGN wavefronts each cover the whole tile and take alternate 16-wide k-steps; their
  // accumulators are added through LDS after the K loop (two wavefronts per SIMD with large wave tiles).
  static constexpr int KSPLIT = KSPLIT_;
  static constexpr int WGM = WGM_, WGN = WGN_, NWG = WGM * WGN, NW = NWG * KSPLIT, NT = NW * 64;
  static constexpr int TM = TILE_M / WGM, TN = TILE_N / WGN, FM = TM / 32, FN = TN / 32;
  static constexpr int BK = BK_;                       // k extent of one ring slot
  static constexpr int NS = NS_;                       // ring slots
  static constexpr int P_BYTES = TILE_M * BK * 2, Q_BYTES = TILE_N * BK * 2;  // operand tiles
  static constexpr int SLOT_BYTES = P_BYTES + Q_BYTES;
  static constexpr int LPT_P = P_BYTES / 1024 / NW;    // direct-to-LDS loads per wavefront per K tile
  static constexpr int LPT_Q = Q_BYTES / 1024 / NW;
  static constexpr int CPR = BK / 8;                   // 16-byte chunks per K-contiguous LDS row
  static constexpr int ROWS_PER_KB = 1024 / (BK * 2);  // K-contiguous rows covered by one 1 KB load
  static_assert(BK == 32 || BK == 64, "ring slot depth");
  static_assert(KSPLIT == 1 || KSPLIT == 2, "at most two K groups");
  static_assert((BK / 16) % (2 * KSPLIT) == 0 || KSPLIT == 1, "each K group needs an even number of k-steps per tile");
  static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be a multiple of the 32 x 32 MFMA");
  static_assert(P_BYTES % (1024 * NW) == 0 && Q_BYTES % (1024 * NW) == 0,
                "tiles must split evenly over the wavefronts' 1 KB loads");
  static_assert(NS * SLOT_BYTES <= 160 * 1024 - 256, "ring exceeds the 160 KB LDS");
};
// MFMA-bound default: 256 x 256 tile, 8 wavefronts (2 per SIMD) of 128 x 64, two 64 KB slots.
#ifndef MI_BIG_WGN
#define MI_BIG_WGN 4
#endif
using CfgBig = FastCfg<256, 2, MI_BIG_WGN, 64, 2>;
// Half-width tile for the last partial round of a GEMM: 256 x 128, wavefronts of 128 x 32.
using CfgHalfN = FastCfg<256, 2, 4, 64, 2, 1, 128>;
// SYRK on ~4096-row Gram matrices: 192 x 192 tiles give 22 * 23 / 2 = 253 lower-triangle tiles, one per
// CU in a single round (256 x 256 tiles would give 136 and leave 47 % of the CUs idle).
// 2 K-groups x 4 wavefronts of 96 x 96, three 48 KB slots (two K tiles in flight).
#ifndef MI_SYRK192_KSPLIT
#define MI_SYRK192_KSPLIT 2
#endif
using CfgSyrk192 = FastCfg<192, 2, 2, 64, 3, MI_SYRK192_KSPLIT>;

// Direct-to-LDS load: every lane fetches 16 bytes from its own global address; the wavefront's 1 KB lands
// at LDS byte address `lds_wave_base` + 16 * lane (the base travels in M0).  Written as inline assembly so
// that completion is tracked only by the explicit s_waitcnt vmcnt(..) in the kernel: the compiler's own
// bookkeeping would make every later LDS read wait for all outstanding loads, i.e. no prefetching.
__device__ __forceinline__ void dma16(const uint16_t* g, char* lds_wave_base) {
  const uint32_t lds_addr = __builtin_amdgcn_readfirstlane(
      (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds_wave_base);  // wave-uniform by construction
#ifndef MI_ABLATE_LOADS
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_addr), "v"(g) : "memory", "m0");
#endif
}

// XOR swizzle of the K-contiguous LDS tile: chunk c of row r is stored at slot kc_slot(r, c) of its row, so
// that the 16 rows a quarter-wave reads (same chunk) cover all 64 banks.
template <int BK>
__device__ __forceinline__ int kc_slot(int row, int c) {
  return BK == 64 ? (c ^ ((row >> 1) & 7)) : (c ^ ((row >> 2) & 3));
}

// Per-thread global pointers of the direct-to-LDS loads of one operand tile.  Rows beyond `rows_valid` are
// redirected to the last valid row: they only feed output rows that the epilogue never stores.
template <class C, bool KS, int ROWS>
struct FastLoader {
  static constexpr int LPT = ROWS * C::BK * 2 / 1024 / C::NW;
  static constexpr int KS_CHUNKS = ROWS / 8;          // 16-byte chunks per k-row of the K-strided layout
  static constexpr int KS_ROWS_PER_KB = 512 / ROWS;   // k-rows covered by one 1 KB load
  const uint16_t* gp[LPT];
  int64_t step;  // elements to advance per K tile

  __device__ __forceinline__ void init(const uint16_t* base, int64_t ld, int row0, int rows_valid, int wave, int lane) {
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      const int b = wave * LPT + i;  // 1 KB block index inside the tile
      if (!KS) {
        const int row = C::ROWS_PER_KB * b + lane / C::CPR;
        const int c = kc_slot<C::BK>(row, lane % C::CPR);  // the swizzle is an involution: slot -> chunk
        int gr = row0 + row;
        gr = gr < rows_valid ? gr : rows_valid - 1;
        gp[i] = base + (int64_t)gr * ld + c * 8;
      } else {
        static_assert(!KS || ROWS == 256 || ROWS == 128, "K-strided LDS layout is laid out for 128/256-wide tiles");
        const int k = KS_ROWS_PER_KB * b + lane / KS_CHUNKS;
        const int c = ((lane % KS_CHUNKS) - 4 * k) & (KS_CHUNKS - 1);
        gp[i] = base + (int64_t)k * ld + row0 + c * 8;
      }
    }
    step = KS ? (int64_t)C::BK * ld : C::BK;
  }
  __device__ __forceinline__ void issue(char* tile, int wave) {
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
      dma16(gp[i], tile + (wave * LPT + i) * 1024);
      gp[i] += step;
    }
  }
};

// MFMA fragment (8 bf16 along k) for 32 consecutive rows starting at `row_base`, k-step q (16 k each).
template <class C, bool KS, int ROWS>
__device__ __forceinline__ bf16x8_t fast_frag(const char* tile, int row_base, int q, int lane) {
  constexpr int KS_CHUNKS = ROWS / 8, KS_ROW_BYTES = ROWS * 2;
  if (!KS) {
    const int row = row_base + (lane & 31);
    const int c = kc_slot<C::BK>(row, 2 * q + (lane >> 5));
    return *reinterpret_cast<const bf16x8_t*>(tile + row * (C::BK * 2) + c * 16);
  } else {
    const int i16 = lane & 15;
    const int col = row_base + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);
    const int kb = 16 * q + 8 * (lane >> 5) + (i16 >> 2);
    s16x4_t lo, hi;
    {
      const int k = kb;
      const int slot = ((col >> 3) + 4 * k) & (KS_CHUNKS - 1);
      lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (s16x4_t __attribute__((address_space(3)))*)(tile + k * KS_ROW_BYTES + slot * 16 + (col & 7) * 2));
    }
    {
      const int k = kb + 4;
      const int slot = ((col >> 3) + 4 * k) & (KS_CHUNKS - 1);
      hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (s16x4_t __attribute__((address_space(3)))*)(tile + k * KS_ROW_BYTES + slot * 16 + (col & 7) * 2));
    }
    typedef short s16x8_t __attribute__((ext_vector_type(8)));
    s16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8_t, both);
  }
}

// Workgroup id -> GEMM tile.  Consecutive workgroup ids are dealt round-robin to the 8 XCDs, each with its
// own L2, so id % 8 names the XCD and id / 8 the position in that XCD's queue.  Each XCD gets a contiguous
// range of tile columns (all tile rows), walked in blocks of XCD_BLOCK_M tile rows: the ~32 tiles an XCD
// works on at one time then form a compact block that shares P row-panels and Q column-panels in L2.
#ifndef MI_XCD_BLOCK_M
#define MI_XCD_BLOCK_M 8
#endif
__device__ __forceinline__ void gemm_tile_of(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
  constexpr int XCDS = 8;
  const int total = tiles_m * tiles_n;
  if (MI_XCD_BLOCK_M == 0 || tiles_n % XCDS != 0 || tiles_m % MI_XCD_BLOCK_M != 0) {
    tm = pid % tiles_m;
    tn = pid / tiles_m;
    return;
  }
  (void)total;
  const int xcd = pid % XCDS, local = pid / XCDS;
  const int cols_per_xcd = tiles_n / XCDS;
  const int block = MI_XCD_BLOCK_M * cols_per_xcd;  // tiles in one row-block of this XCD's column range
  const int rb = local / block, r = local % block;
  tm = rb * MI_XCD_BLOCK_M + r % MI_XCD_BLOCK_M;
  tn = xcd * cols_per_xcd + r / MI_XCD_BLOCK_M;
}

// GEMM-mode epilogue through LDS.  In the MFMA accumulator layout a lane owns one output row and scattered
// 4-column groups, so direct global accesses touch 32 rows per instruction.  Here every wavefront parks one
// 32-row block of its accumulators in its own LDS region (float32, rows padded by 16 bytes against bank
// conflicts), then re-reads it so that 8 consecutive lanes cover 64 consecutive columns of one row: the
// Cin loads and the stores become 16-byte-per-lane, 128-byte-per-row accesses.  No workgroup barrier is
// needed between the passes: a wavefront only touches its own region and LDS operations of one wavefront
// complete in order.
template <class C, bool OUT_F32, bool GUARD>
__device__ __forceinline__ void gemm_epilogue_lds(const GemmParams& p, f32x16_t (&acc)[C::FM][C::FN], char* lds, int wave,
                                                  int lane, int m_base, int n_base, int64_t batch, float alpha,
                                                  float beta, float* red) {
  constexpr int TN = C::TN, ROWB = TN * 4 + 16;
  constexpr int LPR = TN / 8;    // lanes per output row (8 columns each)
  constexpr int RPI = 64 / LPR;  // rows per read iteration
  static_assert(32 % RPI == 0 && 64 % LPR == 0, "wave tile width must be 32, 64 or 128");
  static_assert(C::NW * 32 * ROWB <= C::NS * C::SLOT_BYTES, "epilogue staging exceeds the ring");
  char* reg = lds + wave * (32 * ROWB);
  const int frow = lane & 31, fk = lane >> 5;
  const int rr = lane / LPR, cc = (lane % LPR) * 8;
  const uint16_t* __restrict__ Cb = p.Cin ? p.Cin + batch * p.c_bs : nullptr;
  const bool use_c = beta != 0.0f && Cb != nullptr;
  constexpr int NIT = 32 / RPI;
  // All Cin pieces of this lane are requested up front (the fragment registers of the main loop are dead by
  // now), so the global-load latency is paid once instead of once per piece.
  constexpr bool PREFETCH_ALL = C::FM * NIT * 4 <= 64;  // else one 32-row block at a time (register budget)
  uint4 cin[C::FM][NIT];
  auto load_cin = [&](int i) {
#pragma unroll
    for (int t = 0; t < NIT; ++t) {
      const int m = m_base + i * 32 + t * RPI + rr, n = n_base + cc;
      cin[i][t] = make_uint4(0u, 0u, 0u, 0u);
      if (use_c && (!GUARD || (m < p.M && n < p.N))) cin[i][t] = *reinterpret_cast<const uint4*>(Cb + (int64_t)m * p.ldc + n);
    }
  };
  if (PREFETCH_ALL) {
#pragma unroll
    for (int i = 0; i < C::FM; ++i) load_cin(i);
  }
  float ssq = 0.0f;
#pragma unroll
  for (int i = 0; i < C::FM; ++i) {
    if (!PREFETCH_ALL) load_cin(i);
#pragma unroll
    for (int j = 0; j < C::FN; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4_t v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
        *reinterpret_cast<f32x4_t*>(reg + frow * ROWB + (j * 32 + 8 * g + 4 * fk) * 4) = v;
      }
#pragma unroll
    for (int t = 0; t < NIT; ++t) {
      const int row = t * RPI + rr;
      const int m = m_base + i * 32 + row, n = n_base + cc;
      f32x4_t lo = *reinterpret_cast<const f32x4_t*>(reg + row * ROWB + cc * 4);
      f32x4_t hi = *reinterpret_cast<const f32x4_t*>(reg + row * ROWB + cc * 4 + 16);
      if (GUARD && (m >= p.M || n >= p.N)) continue;
      lo *= alpha;
      hi *= alpha;
      if (use_c) {
        const uint32_t w[4] = {cin[i][t].x, cin[i][t].y, cin[i][t].z, cin[i][t].w};
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          lo[2 * e] = __builtin_fmaf(beta, __uint_as_float(w[e] << 16), lo[2 * e]);
          lo[2 * e + 1] = __builtin_fmaf(beta, __uint_as_float(w[e] & 0xffff0000u), lo[2 * e + 1]);
          hi[2 * e] = __builtin_fmaf(beta, __uint_as_float(w[2 + e] << 16), hi[2 * e]);
          hi[2 * e + 1] = __builtin_fmaf(beta, __uint_as_float(w[2 + e] & 0xffff0000u), hi[2 * e + 1]);
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) ssq = __builtin_fmaf(lo[e], lo[e], __builtin_fmaf(hi[e], hi[e], ssq));
      if (OUT_F32) {
        float* o = reinterpret_cast<float*>(p.Out) + batch * p.o_bs + (int64_t)m * p.ldo + n;
        *reinterpret_cast<f32x4_t*>(o) = lo * p.out_scale;
        *reinterpret_cast<f32x4_t*>(o + 4) = hi * p.out_scale;
      } else {
        uint16_t* o = reinterpret_cast<uint16_t*>(p.Out) + batch * p.o_bs + (int64_t)m * p.ldo + n;
        const uint2 a = __builtin_bit_cast(uint2, __builtin_convertvector(lo, bf16x4_t));
        const uint2 b = __builtin_bit_cast(uint2, __builtin_convertvector(hi, bf16x4_t));
        *reinterpret_cast<uint4*>(o) = make_uint4(a.x, a.y, b.x, b.y);
      }
    }
  }
  if (p.slots_out != nullptr) {
    const float total = block_sum_f32<C::NT>(ssq, red);
    if (threadIdx.x == 0) p.slots_out[batch * p.slot_stride + p.slot_base + blockIdx.x] = total;
  }
}

// s_waitcnt immediate for gfx9: vmcnt in bits [3:0] and [15:14], expcnt [6:4] = 7 (no wait), lgkmcnt [11:8].
constexpr int waitcnt_imm(int vmcnt, int lgkmcnt) {
  return (vmcnt & 15) | ((vmcnt >> 4) << 14) | 0x70 | ((lgkmcnt & 15) << 8);
}

template <class C, bool P_KS, bool Q_KS, int MODE, bool OUT_F32, bool EDGE>
__global__ void __launch_bounds__(C::NT) gemm_fast_kernel(GemmParams p) {
  constexpr int NS = C::NS, FM = C::FM, FN = C::FN, P_BYTES = C::P_BYTES, NT = C::NT;
  // One array per ring slot: every LDS access below names its slot statically.
  __shared__ __align__(1024) char ring[NS][C::SLOT_BYTES];
  __shared__ float red[NT / 64];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: everything derived from it stays in SGPRs
  const int kgroup = wave / C::NWG, wig = wave % C::NWG;  // K group and position inside it
  const int wm = wig % C::WGM, wn = wig / C::WGM;
  const int64_t batch = blockIdx.y;
  int tm, tn;
  if (MODE == MODE_SYRK) {
    // The grid is padded to a multiple of 8 workgroups: id % 8 names the XCD (round-robin dispatch), and
    // each XCD takes one contiguous chunk of the blocked triangular enumeration.
    const int total = p.tiles_m * (p.tiles_m + 1) / 2;
    const int per_xcd = (int)gridDim.x / 8;
    const int s = ((int)blockIdx.x % 8) * per_xcd + (int)blockIdx.x / 8;
    if (s >= total) return;  // padding workgroup (whole workgroup leaves before any barrier)
    tri_block_decode(s, p.tiles_m, tm, tn);
  } else {
    gemm_tile_of((int)blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
  }
  const int m0 = tm * C::TILE_M, n0 = tn * C::TILE_N;

  FastLoader<C, P_KS, C::TILE_M> lp;
  FastLoader<C, Q_KS, C::TILE_N> lq;
  lp.init(p.P + batch * p.p_bs, p.ldp, m0, p.M, wave, lane);
  lq.init(p.Q + batch * p.q_bs, p.ldq, n0, p.N, wave, lane);

  f32x16_t acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  const int nk = p.K / C::BK;
  constexpr int NQ = C::BK / 16 / C::KSPLIT;  // k-steps of one tile that this wavefront multiplies
  constexpr int LOADS_PER_TILE = C::LPT_P + C::LPT_Q;  // per thread, both operands
  static_assert(NQ % 2 == 0, "fragment buffer parity assumes an even number of k-steps per tile");
  static_assert((NS - 2) * LOADS_PER_TILE < 64, "vmcnt is a 6-bit counter");

  // Pipeline.  Ring slot kt % NS holds K tile kt.  While tile kt is multiplied, tiles kt+1 .. kt+NS-1 are in
  // flight; the slot refilled at the top of tile kt is the one tile kt-1 occupied, which every wavefront left
  // before the previous barrier.  Fragment registers are double buffered (the LDS reads of k-step q+1 run
  // under the MFMAs of k-step q), and the barrier that publishes tile kt+1 sits before the last k-step of
  // tile kt so that its skew and the first fragment reads of tile kt+1 are covered by that k-step's MFMAs.
#ifdef MI_TIMING
  long long t_load = 0, t_bar = 0;
#endif
  bf16x8_t fp[2][FM], fq[2][FN];
  auto fetch = [&](const char* st, int q, int buf) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
      fp[buf][i] = fast_frag<C, P_KS, C::TILE_M>(st, wm * C::TM + i * 32, q * C::KSPLIT + kgroup, lane);
#pragma unroll
    for (int j = 0; j < FN; ++j)
      fq[buf][j] = fast_frag<C, Q_KS, C::TILE_N>(st + P_BYTES, wn * C::TN + j * 32, q * C::KSPLIT + kgroup, lane);
  };
  auto mma = [&](int buf) {
#ifdef MI_SETPRIO
    __builtin_amdgcn_s_setprio(MI_SETPRIO);
#endif
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fq[buf][j], fp[buf][i], acc[i][j], 0, 0, 0);
#ifdef MI_SETPRIO
    __builtin_amdgcn_s_setprio(0);
#endif
  };
  auto issue = [&](char* slot) {
    lp.issue(slot, wave);
    lq.issue(slot + P_BYTES, wave);
  };
  auto k_tile = [&](int kt, char* cur, char* nxt, char* refill) {
    const bool refilled = kt + NS - 1 < nk;
    if (refilled) issue(refill);  // tile kt+NS-1 -> slot (kt-1) % NS
#pragma unroll
    for (int q = 0; q + 1 < NQ; ++q) {
      fetch(cur, q + 1, (q + 1) & 1);
      mma(q & 1);
#ifndef MI_NO_SCHED_INTERLEAVE
      // one LDS read issued in the shadow of every MFMA
      constexpr int READS = FM * (P_KS ? 2 : 1) + FN * (Q_KS ? 2 : 1);
      constexpr int MMAS = FM * FN;
#pragma unroll
      for (int x = 0; x < MMAS; ++x) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, (READS + MMAS - 1) / MMAS, 0);
      }
#endif
    }
    // own loads of tile kt+1 have landed (younger tiles may stay in flight); own reads of `cur` are done
#ifdef MI_TIMING
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));
    const long long tw0 = __builtin_readcyclecounter();
#endif
    if (refilled)
      __builtin_amdgcn_s_waitcnt(waitcnt_imm((NS - 2) * LOADS_PER_TILE, 0));
    else
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
#ifdef MI_TIMING
    const long long tw1 = __builtin_readcyclecounter();
#endif
#ifndef MI_ABLATE_BARRIER
    __syncthreads();
#endif
#ifdef MI_TIMING
    const long long tw2 = __builtin_readcyclecounter();
    t_load += tw1 - tw0;
    t_bar += tw2 - tw1;
#endif
    if (kt + 1 < nk) fetch(nxt, 0, 0);
    mma((NQ - 1) & 1);
  };

#ifdef MI_TIMING
  const long long t_start = __builtin_readcyclecounter();
#endif
  // prologue: tiles 0 .. NS-2 in flight, wait for tile 0
#pragma unroll
  for (int t = 0; t < NS - 1; ++t)
    if (t < nk) issue(ring[t]);
  if (nk >= NS - 1)
    __builtin_amdgcn_s_waitcnt(waitcnt_imm((NS - 2) * LOADS_PER_TILE, 15));
  else
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
  __syncthreads();
  fetch(ring[0], 0, 0);
  for (int kt = 0; kt < nk; kt += NS) {
#pragma unroll
    for (int u = 0; u < NS; ++u)
      if (kt + u < nk) k_tile(kt + u, ring[u], ring[(u + 1) % NS], ring[(u + NS - 1) % NS]);
  }

  if constexpr (C::KSPLIT == 2) {
    // Sum the two K groups: group 1 parks its accumulators in the ring (lane-linear, conflict free),
    // group 0 adds them and carries on with the epilogue alone.
    static_assert(C::KSPLIT == 1 || C::NWG * FM * FN * 4096 <= NS * C::SLOT_BYTES, "accumulators exceed the ring");
    __syncthreads();  // all fragment reads of the ring are done
    char* park = &ring[0][0] + wig * (FM * FN * 4096);
    if (kgroup == 1) {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            f32x4_t v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
            *reinterpret_cast<f32x4_t*>(park + ((i * FN + j) * 4 + g) * 1024 + lane * 16) = v;
          }
    }
    __syncthreads();
    if (kgroup == 0) {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const f32x4_t v = *reinterpret_cast<const f32x4_t*>(park + ((i * FN + j) * 4 + g) * 1024 + lane * 16);
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][4 * g + r] += v[r];
          }
    }
  }
#ifdef MI_TIMING
  const long long t_loop = __builtin_readcyclecounter();
#endif
  float beta = p.beta;
  const float shift = resolve_shift<NT>(p, batch, red, beta);
  const bool diag = (MODE == MODE_SYRK) && (tm == tn);
  if constexpr (MODE == MODE_GEMM && (C::TN == 32 || C::TN == 64 || C::TN == 128)) {
    __syncthreads();  // every wavefront has finished reading the ring: it can be reused as staging space
    gemm_epilogue_lds<C, OUT_F32, EDGE>(p, acc, &ring[0][0], wave, lane, m0 + wm * C::TM, n0 + wn * C::TN, batch, p.alpha,
                                        beta, red);
  } else {
    static_assert(C::KSPLIT == 1 || MODE == MODE_SYRK, "the K-group variant is wired for SYRK only");
    // (SYRK never takes the per-workgroup sum at the end of tile_epilogue, so group 1 may simply skip it)
    if (C::KSPLIT == 1 || kgroup == 0)
      tile_epilogue<MODE, OUT_F32, EDGE, FM, FN, NT>(p, acc, m0 + wm * C::TM, n0 + wn * C::TN, lane, batch, diag, p.alpha,
                                                     beta, shift, red);
  }
#ifdef MI_TIMING
  if (p.slots_in && lane == 0) {  // debug build only: slots_in doubles as the timing dump
    __builtin_amdgcn_s_waitcnt(0);
    const long long t_end = __builtin_readcyclecounter();
    long long* dump = (long long*)p.slots_in + ((long long)blockIdx.x * C::NW + wave) * 4;
    dump[0] = t_load;
    dump[1] = t_bar;
    dump[2] = t_loop - t_start;
    dump[3] = t_end - t_loop;
  }
#endif
}

}  // namespace mi
