// Fast path of the bf16 tile engine for the MFMA-bound shapes (K % 64 == 0, no K tail; row edges are
// allowed and handled by clamped loads plus a guarded epilogue).
//
// A variant is described by FastCfg: workgroup tile (TILE_M x TILE_N), wavefront grid, ring-slot depth BK, number
// of ring slots and the MFMA shape.  Global -> LDS goes through the direct-to-LDS load (16 bytes per lane, a
// wavefront fills 1 KB of LDS at base + 16 * lane); the slots form a ring with one barrier per K tile (see the
// kernel).  Because LDS placement is fixed by the lane id, swizzling is done by choosing which global chunk a lane
// fetches:
//   K-contiguous operand: LDS row = 128 B (8 chunks); chunk c of row r sits at slot c ^ ((r >> 1) & 7),
//     so the 16 rows one pass of a ds_read_b128 reads cover all 64 banks.
//   K-strided operand: LDS row = one k (ROWS values); chunk c of row k sits at slot (c + ks_rot(k)) mod chunks;
//     fragments are fetched with the LDS transpose read ds_read_b64_tr_b16, which returns to lane i of a 16-lane
//     group the four k-values of row i from four consecutive k-rows.
// tests/test_lds_layout_model.py restates loader and fragment reads on the host and checks them against each other.
#pragma once
#include <type_traits>
#include <utility>

#include "gemm_engine.hpp"

// Address arithmetic that the kernels share with the host-side bounds check (host_check.hpp): plain integer
// functions, compiled for both sides, so that what the check replays is the code the GPU runs.
#define MI_HD __host__ __device__ __forceinline__

namespace mi {

typedef short s16x4_t __attribute__((ext_vector_type(4)));

// Compile-time loop: f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N - 1>{}).  Used where a
// body must be unrolled whatever its size (register arrays indexed by the loop variable must never become
// runtime-indexed, i.e. scratch memory).
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// Compile-time shape of one fast-kernel variant.  The MFMA is v_mfma_f32_16x16x32_bf16 throughout: of the two bf16
// shapes (same peak) it moves a quarter of the accumulator registers per instruction and draws less power per FLOP
// on random operands, which is what bounds the clock on this part.
template <int TILE_M_, int WGM_, int WGN_, int BK_, int NS_, int TILE_N_ = TILE_M_>
struct FastCfg {
  static constexpr int MI = 16, KI = 32;                     // MFMA tile rows / k per MFMA
  static constexpr int TILE_M = TILE_M_, TILE_N = TILE_N_;  // workgroup tile: rows of P x rows of Q
  static constexpr int TILE = TILE_M_;                      // (SYRK uses square tiles)
  static constexpr int WGM = WGM_, WGN = WGN_, NW = WGM * WGN, NT = NW * 64;
  static constexpr int TM = TILE_M / WGM, TN = TILE_N / WGN, FM = TM / MI, FN = TN / MI;
  static constexpr int BK = BK_;                       // k extent of one ring slot
  static constexpr int NS = NS_;                       // ring slots
  static constexpr int P_BYTES = TILE_M * BK * 2, Q_BYTES = TILE_N * BK * 2;  // operand tiles
  static constexpr int SLOT_BYTES = P_BYTES + Q_BYTES;
  static constexpr int LPT_P = P_BYTES / 1024 / NW;    // direct-to-LDS loads per wavefront per K tile
  static constexpr int LPT_Q = Q_BYTES / 1024 / NW;
  static constexpr int CPR = BK / 8;                   // 16-byte chunks per K-contiguous LDS row
  static constexpr int ROWS_PER_KB = 1024 / (BK * 2);  // K-contiguous rows covered by one 1 KB load
  static_assert(BK == 32 || BK == 64, "ring slot depth");
  static_assert((BK / KI) % 2 == 0, "an even number of k-steps per tile");
  static_assert(TM % MI == 0 && TN % MI == 0, "wave tile must be a multiple of the MFMA tile");
  static_assert(P_BYTES % (1024 * NW) == 0 && Q_BYTES % (1024 * NW) == 0,
                "tiles must split evenly over the wavefronts' 1 KB loads");
  static_assert(NS * SLOT_BYTES <= 160 * 1024 - 256, "ring exceeds the 160 KB LDS");
};
// One wavefront per SIMD (4 per workgroup), accumulators in 256 / 128 / 144 registers.
// Batched small matrices (per-head shapes, 128 rows): GEMM+AXPY tile 128 x 256 (wavefronts of 128 x 64) and a
// 128 x 128 tile (wavefronts of 64 x 64) for the split-K Gram partials.
using CfgM128 = FastCfg<128, 1, 4, 64, 2, 256>;
using CfgT128 = FastCfg<128, 2, 2, 64, 3, 128>;
// The same tile with a two-slot ring (64 KB): two workgroups share a CU, so one's epilogue overlaps the other's K loop.
using CfgT128x2 = FastCfg<128, 2, 2, 64, 2, 128>;
using CfgBig = FastCfg<256, 2, 2, 64, 2, 256>;      // wavefronts of 128 x 128
using CfgHalfN = FastCfg<256, 2, 2, 64, 3, 128>;    // wavefronts of 128 x 64
using CfgSyrk192 = FastCfg<192, 2, 2, 64, 3, 192>;  // wavefronts of 96 x 96


// Rotation (in 16-byte chunks) of k-row k of a K-strided LDS tile, chosen so that the k-rows which one pass of the
// transpose read touches (32 lanes: 4 k-rows x 32 B at k and at k + 8) fall on disjoint banks: 32 B per k inside an
// 8-row group, 128 B per group.
MI_HD int ks_rot(int k) { return 2 * (k & 7) + 8 * (k >> 3); }

// Direct-to-LDS load: every lane fetches 16 bytes from its own global address; the wavefront's 1 KB lands
// at LDS byte address `lds_addr` + 16 * lane (`lds_addr` is wave-uniform and travels in M0).  Written as inline assembly so
// that completion is tracked only by the explicit s_waitcnt vmcnt(..) in the kernel: the compiler's own
// bookkeeping would make every later LDS read wait for all outstanding loads, i.e. no prefetching.
// (M0 is a reserved register: the compiler never keeps a value in it across statements, so it is not
// listed as clobbered.)
__device__ __forceinline__ void dma16(const uint16_t* g, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_addr), "v"(g) : "memory");
}

// 16-byte global store at device scope (sc1): the line is written through the XCD's L2 as it is stored, instead of
// staying dirty there until the write-back at the end of the kernel (a 4096 x 4096 bf16 result leaves 33.5 MB in the
// eight L2s; written through, the tail of every launch is shorter: -1.3 .. -1.7 % per Newton-Schulz call, A/B on one
// box).  Inline assembly, because no builtin sets the scope bit of a plain store.  The compiler does not know that
// this is a store of more than 8 bytes, whose data registers must not be written by a VALU instruction in the next
// two wait states, so the wait states are part of the statement (without them the 256 x 256 tile stored a few
// per cent wrong values: the registers were refilled for the next store right behind this one).
// Used by the lower-triangle epilogue only: the float32 write-out of the GEMM mode, 32 bytes per lane in two pieces,
// became 24 % slower with it (390 -> 482 us at 4096 x 14336), its bf16 write-out did not change.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void store16_through(void* ptr, const uint4& v) {
  const u32x4_t w = {v.x, v.y, v.z, v.w};
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(ptr), "v"(w) : "memory");
}

// XOR swizzle of the K-contiguous LDS tile: chunk c of row r is stored at slot kc_slot(r, c) of its row, so
// that the 16 rows a quarter-wave reads (same chunk) cover all 64 banks.
template <int BK>
MI_HD int kc_slot(int row, int c) {
  return BK == 64 ? (c ^ ((row >> 1) & 7)) : (c ^ ((row >> 2) & 3));
}

// Same load with the address split into a wave-uniform 64-bit base (SGPR pair) and a per-lane 32-bit byte
// offset: the blocks of one tile differ only in the base, so a handful of offset registers serve all loads
// of an operand and the per-load address arithmetic runs on the scalar unit.
__device__ __forceinline__ void dma16_sv(uint64_t sbase, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}

// Direct-to-LDS loads of one operand tile (ROWS rows of the operand x BK along k).  The tile is cut into
// 1 KB blocks, LPT per wavefront; block b = wave * LPT + i lands at tile + 1024 * b.
//   CLAMP = false: the tile lies wholly inside the operand.  Block b starts at a wave-uniform address and the
//     lanes' offsets inside a block repeat with a short period in b (the swizzle phase), so the loader keeps
//     one scalar base plus NV lane-offset registers.
//   CLAMP = true: rows beyond `rows_valid` are redirected to the last valid row (they only feed output rows
//     that the epilogue never stores); every load keeps its own lane-offset register (32 bits, relative to the
//     first row of the tile: the launcher refuses leading dimensions for which TILE rows do not fit), the base
//     is the same scalar as above.  (With a 64-bit pointer per load, advanced by vector adds in every K tile, the
//     lower-triangle product of 4096 rows -- 192 does not divide them -- was 3 % slower than that of 4224 rows.)
template <class C, bool KS, int ROWS, bool CLAMP>
struct FastLoader {
  static constexpr int LPT = ROWS * C::BK * 2 / 1024 / C::NW;
  static constexpr int KS_CHUNKS = ROWS / 8;          // 16-byte chunks per k-row of the K-strided layout
  static constexpr int KS_ROWS_PER_KB = 512 / ROWS;   // k-rows covered by one 1 KB load
  // period of the swizzle phase in the block index
  static constexpr int PERIOD = KS ? (KS_CHUNKS / KS_ROWS_PER_KB > 0 ? KS_CHUNKS / KS_ROWS_PER_KB : 1) : (C::BK == 64 ? 2 : 1);
  static constexpr bool PERIODIC = LPT % PERIOD == 0;  // then the phase of load i is i % PERIOD for every wavefront
  static constexpr int NV = CLAMP ? LPT : (PERIODIC ? (PERIOD < LPT ? PERIOD : LPT) : LPT);
  static_assert(!KS || ROWS == 256 || ROWS == 128, "K-strided LDS layout is laid out for 128/256-wide tiles");
  // (a K-strided tile at the edge of its operand would need clamping along the contiguous dimension, which a
  // 16-byte load cannot do per element: the launcher never sends such a tile here)
  static_assert(!(KS && CLAMP), "edge tiles of K-strided operands are not served by the fast kernel");

  uint32_t voff[NV];                    // per-lane byte offsets: inside a block (!CLAMP), from the tile's first row (CLAMP)
  uint64_t base;                        // byte address of this wavefront's first block (!CLAMP) or of the tile (CLAMP); uniform
  int64_t block_step;                   // !CLAMP: bytes between consecutive blocks (uniform)
  int64_t step;                         // advance per K tile in bytes

  // lane's element offset inside block b, relative to the block's first element
  static MI_HD int64_t lane_part(int b, int64_t ld, int lane) {
    if (!KS) {
      const int lr = lane / C::CPR;
      const int c = kc_slot<C::BK>(C::ROWS_PER_KB * b + lr, lane % C::CPR);  // the swizzle is an involution
      return (int64_t)lr * ld + c * 8;
    } else {
      const int kr = lane / KS_CHUNKS;
      const int c = ((lane % KS_CHUNKS) - ks_rot(KS_ROWS_PER_KB * b + kr)) & (KS_CHUNKS - 1);
      return (int64_t)kr * ld + c * 8;
    }
  }

  MI_HD void init(const uint16_t* opbase, int64_t ld, int row0, int rows_valid, int wave, int lane) {
    if constexpr (CLAMP) {
#pragma unroll
      for (int i = 0; i < LPT; ++i) {
        const int b = wave * LPT + i;  // 1 KB block index inside the tile
        const int row = C::ROWS_PER_KB * b + lane / C::CPR;
        const int c = kc_slot<C::BK>(row, lane % C::CPR);
        int gr = row0 + row;
        gr = gr < rows_valid ? gr : rows_valid - 1;
        voff[i] = (uint32_t)(2 * ((int64_t)(gr - row0) * ld + c * 8));
      }
      base = (uint64_t)(uintptr_t)(opbase + (int64_t)row0 * ld);
      block_step = 0;
      step = 2 * (int64_t)C::BK;
    } else {
      const int b0 = wave * LPT;
#pragma unroll
      for (int v = 0; v < NV; ++v) voff[v] = (uint32_t)(2 * lane_part(PERIODIC ? v : b0 + v, ld, lane));
      const int64_t first = KS ? (int64_t)(KS_ROWS_PER_KB * b0) * ld + row0 : (int64_t)(row0 + C::ROWS_PER_KB * b0) * ld;
      base = (uint64_t)(uintptr_t)(opbase + first);
      block_step = 2 * (int64_t)(KS ? KS_ROWS_PER_KB : C::ROWS_PER_KB) * ld;
      step = 2 * (KS ? (int64_t)C::BK * ld : (int64_t)C::BK);
    }
  }
  // Load i (0 .. LPT-1) of the current K tile reads 16 bytes at scalar_base(i) + lane_offset(i).
  MI_HD uint64_t scalar_base(int i) const { return CLAMP ? base : base + (uint64_t)(i * block_step); }
  MI_HD uint32_t lane_offset(int i) const { return voff[CLAMP ? i : (PERIODIC ? i % NV : i)]; }
  MI_HD uint64_t address(int i) const { return scalar_base(i) + lane_offset(i); }
  // Issues load i of the current K tile; `lds_tile` is the LDS byte address of the operand tile in the target ring
  // slot.  advance() moves on to the next K tile once all LPT loads are out.
  __device__ __forceinline__ void issue_one(uint32_t lds_tile, int wave, int i) {
    dma16_sv(scalar_base(i), lane_offset(i), lds_tile + (wave * LPT + i) * 1024);
  }
  MI_HD void advance() { base += step; }
};

// MFMA fragment (8 bf16 along k per lane) of a K-contiguous tile for 16 consecutive rows starting at `row_base`,
// k-step q (32 k each): lane l -> row l % 16, k = 32 q + 8 (l / 16) .. +7.
template <class C>
__device__ __forceinline__ bf16x8_t fast_frag(const char* tile, int row_base, int q, int lane) {
  const int row = row_base + (lane & 15);
  const int c = kc_slot<C::BK>(row, (C::KI / 8) * q + (lane >> 4));
  return *reinterpret_cast<const bf16x8_t*>(tile + row * (C::BK * 2) + c * 16);
}

// K-strided tiles are read with the LDS transpose read: its 16 lanes fetch 4 k-rows x 16 rows (8 bytes per lane: 4
// consecutive rows at one k) and every lane receives the 4 k-values of its own row.  The fragment is formed from two
// per-lane constants (see ks16_consts): the LDS address of every transpose read is ((S + c) & rowmask | R) + constant, i.e. two VALU operations next to the read instead
// of one address register per (fragment, k-half, k-step, ring slot) kept alive across the whole K loop.
template <int ROWS>
__device__ __forceinline__ void ks16_consts(int lane, int wave_row_base, uint32_t& S, uint32_t& R) {
  const int g = lane >> 4, i16 = lane & 15, kk = i16 >> 2, cq = i16 & 3;
  S = (uint32_t)((wave_row_base / 8 + (cq >> 1) + 2 * kk + 8 * g) * 16 + (cq & 1) * 8);
  R = (uint32_t)((8 * g + kk) * (ROWS * 2));
}
template <int ROWS>
__device__ __forceinline__ bf16x8_t fast_frag16_ks(uint32_t tile_lds, uint32_t S, uint32_t R, int r, int q) {
  constexpr int ROWB = ROWS * 2;  // bytes per k-row = 16 * chunks per k-row (a power of two)
  static_assert((ROWB & (ROWB - 1)) == 0, "row mask");
  typedef s16x4_t __attribute__((address_space(3))) * lds_ptr;
  const uint32_t a0 = (((S + (uint32_t)(2 * r) * 16u) & (ROWB - 1)) | R) + tile_lds + (uint32_t)(32 * q) * ROWB;
  const uint32_t a1 = (((S + (uint32_t)(2 * r + 8) * 16u) & (ROWB - 1)) | R) + tile_lds + (uint32_t)(32 * q + 4) * ROWB;
  const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(uintptr_t)a0);
  const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(uintptr_t)a1);
  return __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

// acc += A B with the accumulator tied in place (AGPRs).  With the builtin the register allocator is free to
// give the result other registers than the addend and then restores the loop-carried layout with copies.
// The compiler does not see an MFMA here: code that reads the accumulators with VALU instructions must be
// separated from the last of these by mfma_drain().
__device__ __forceinline__ void mfma16_inplace(f32x4_t& c, const bf16x8_t& a, const bf16x8_t& b) {
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
// (The scheduling barriers keep the compiler from moving a register copy of an accumulator, which is no memory
// access and so not ordered by the clobber, from behind the wait states to in front of them.)
__device__ __forceinline__ void mfma_drain() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

// Workgroup id -> GEMM tile.  Consecutive workgroup ids are dealt round-robin to the 8 XCDs, each with its
// own L2, so id % 8 names the XCD and id / 8 the position in that XCD's queue.  Each XCD gets a contiguous
// range of tile columns (all tile rows), walked in blocks of XCD_BLOCK_M tile rows: the ~32 tiles an XCD
// works on at one time then form a compact block that shares P row-panels and Q column-panels in L2.
constexpr int XCD_BLOCK_M = 8;
MI_HD void gemm_tile_of(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
  constexpr int XCDS = 8;
  if (tiles_n % XCDS != 0 || tiles_m % XCD_BLOCK_M != 0) {
    tm = pid % tiles_m;
    tn = pid / tiles_m;
    return;
  }
  const int xcd = pid % XCDS, local = pid / XCDS;
  const int cols_per_xcd = tiles_n / XCDS;
  const int block = XCD_BLOCK_M * cols_per_xcd;  // tiles in one row-block of this XCD's column range
  const int rb = local / block, r = local % block;
  tm = rb * XCD_BLOCK_M + r % XCD_BLOCK_M;
  tn = xcd * cols_per_xcd + r / XCD_BLOCK_M;
}

// GEMM-mode epilogue through LDS.  In the MFMA accumulator layout a lane owns one output row and scattered
// 4-column groups, so direct global accesses touch 32 rows per instruction.  Here every wavefront parks one
// 32-row block of its accumulators in its own LDS region (float32, rows padded by 16 bytes against bank
// conflicts), then re-reads it so that 8 consecutive lanes cover 64 consecutive columns of one row: the
// Cin loads and the stores become 16-byte-per-lane, 128-byte-per-row accesses.  (MI = rows of one MFMA tile.)
// No workgroup barrier is needed between the passes: a wavefront only touches its own region and LDS operations of one wavefront
// complete in order.
// Transposed float32 output (p.out_transposed): the finished values go back to the staging rows and are read a
// second time down the columns, a lane taking four consecutive rows of one column (16 bytes of the transposed
// matrix, the sixteen rows of the block 64 bytes); row pitch mod 64 words is 4, so the 64 lanes of such a read fall
// on 64 different banks.
// RMW: the kernel variant for p.out_accum != 0, a compile-time flag so that the plain write-out carries none of its
// registers and branches (with a run-time flag the plain float32 product of 4096 x 14336 took 7 us longer).
// Geometry of the staged GEMM epilogue, relative to the first row and column of the wavefront's block.
template <class C>
struct GemmStage {
  static constexpr int TN = C::TN, MI = C::MI;
  static constexpr int LPR = TN / 8;    // lanes per output row (8 columns each)
  static constexpr int RPI = 64 / LPR;  // rows per read iteration
  static constexpr int NIT = MI / RPI;
  static_assert(MI % RPI == 0 && 64 % LPR == 0, "wave tile width must be 32, 64 or 128");
  // Row-wise passes (addend loads, old values, stores): piece t of 16-row block i of a lane is 8 columns of one row.
  static MI_HD void piece_of(int lane, int i, int t, int& dm, int& dn) {
    dm = i * MI + t * RPI + lane / LPR;
    dn = (lane % LPR) * 8;
  }
  // Transposed float32 write-out: piece t of block i of a lane is four consecutive rows of one column.
  static MI_HD void transposed_piece_of(int lane, int i, int t, int& dm, int& dn) {
    dm = i * MI + 4 * (lane >> 4);
    dn = 16 * t + (lane & 15);
  }
};

template <class C, bool OUT_F32, bool GUARD, bool RMW>
__device__ __forceinline__ void gemm_epilogue_lds(const GemmParams& p, f32x4_t (&acc)[C::FM][C::FN], char* lds, int wave,
                                                  int lane, int m_base, int n_base, int64_t batch, float alpha,
                                                  float beta, float* red) {
  using G = GemmStage<C>;
  constexpr int TN = C::TN, ROWB = TN * 4 + 16, MI = C::MI;
  constexpr int LPR = G::LPR, RPI = G::RPI;
  static_assert(C::NW * MI * ROWB <= C::NS * C::SLOT_BYTES, "epilogue staging exceeds the ring");
  // two staging regions per wavefront when the ring has room: block i+1 is parked while block i is still being
  // re-read and stored
  constexpr int NREG = 2 * C::NW * MI * ROWB <= C::NS * C::SLOT_BYTES ? 2 : 1;
  const int frow = lane & (MI - 1), fk = lane / MI;
  const int rr = lane / LPR, cc = (lane % LPR) * 8;
  const uint16_t* __restrict__ Cb = p.Cin ? p.Cin + batch * p.c_bs : nullptr;
  const bool use_c = beta != 0.0f && Cb != nullptr;
  constexpr int NIT = MI / RPI;
  // All Cin pieces of this lane are requested up front (the fragment registers of the main loop are dead by
  // now), so the global-load latency is paid once instead of once per piece.
  // (register budget: a workgroup of four wavefronts leaves each lane 512 registers, 256 of them free here)
  constexpr bool PREFETCH_ALL = C::FM * NIT * 4 <= (C::NW <= 4 ? 160 : 64);  // else one MI-row block at a time
  // blocks in flight (a block's registers are refilled when it has been consumed); the in-place variant of a large tile
  // shares the registers with the old values
  constexpr int CW = !PREFETCH_ALL ? 1 : ((RMW && C::FM * NIT * 4 > 64 && C::FM > 4) ? 4 : C::FM);
  uint4 cin[CW][NIT];
  auto load_cin = [&](int i) {
#pragma unroll
    for (int t = 0; t < NIT; ++t) {
      int dm, dn;
      G::piece_of(lane, i, t, dm, dn);
      const int m = m_base + dm, n = n_base + dn;
      cin[i % CW][t] = make_uint4(0u, 0u, 0u, 0u);
      if (use_c && (!GUARD || (m < p.M && n < p.N))) cin[i % CW][t] = *reinterpret_cast<const uint4*>(Cb + (int64_t)m * p.ldc + n);
    }
  };
#pragma unroll
  for (int i = 0; i < CW && i < C::FM; ++i) load_cin(i);
  // In-place update of a float32 matrix (out_accum != 0): the old values of a 16-row block are requested one block
  // ahead (loaded where they are used, every one of the FM * NIT pieces waits out a memory latency of its own:
  // measured 22 us per 256 x 256 tile against 12 this way).
  constexpr int OW = 2;  // blocks in flight (three and four: no faster, and the 256 x 256 tile starts to spill)
  // (A kernel of its own, not two copies of the epilogue behind a branch in one kernel: that made the 256 x 256 tile
  // spill 548 bytes per lane.)
  static_assert(!RMW || OUT_F32, "in-place update of a float32 matrix");
  const bool rmw_t = RMW && !GUARD && p.out_transposed;
  f32x4_t oldv[RMW ? OW : 1][RMW ? (NIT * 2 > TN / 16 ? NIT * 2 : TN / 16) : 1];
  auto load_old = [&](int i) {
    if constexpr (RMW) {
      if (rmw_t) {
#pragma unroll
        for (int t = 0; t < TN / 16; ++t) {
          int dm, dn;
          G::transposed_piece_of(lane, i, t, dm, dn);
          oldv[i % OW][t] = *reinterpret_cast<const f32x4_t*>(
              reinterpret_cast<const float*>(p.Out) + batch * p.o_bs + (int64_t)(n_base + dn) * p.ldo + m_base + dm);
        }
      } else {
#pragma unroll
        for (int t = 0; t < NIT; ++t) {
          int dm, dn;
          G::piece_of(lane, i, t, dm, dn);
          const int m = m_base + dm, n = n_base + dn;
          if (GUARD && (m >= p.M || n >= p.N)) continue;
          const float* o = reinterpret_cast<const float*>(p.Out) + batch * p.o_bs + (int64_t)m * p.ldo + n;
          oldv[i % OW][2 * t] = *reinterpret_cast<const f32x4_t*>(o);
          oldv[i % OW][2 * t + 1] = *reinterpret_cast<const f32x4_t*>(o + 4);
        }
      }
    }
  };
#pragma unroll
  for (int i = 0; RMW && i < OW && i < C::FM; ++i) load_old(i);
  float ssq = 0.0f;
#pragma unroll
  for (int i = 0; i < C::FM; ++i) {
    char* reg = lds + (wave * NREG + i % NREG) * (MI * ROWB);
#pragma unroll
    for (int j = 0; j < C::FN; ++j)
{
        const f32x4_t v = acc[i][j];
        *reinterpret_cast<f32x4_t*>(reg + frow * ROWB + (j * MI + 4 * fk) * 4) = v;
      }
#pragma unroll
    for (int t = 0; t < NIT; ++t) {
      const int row = t * RPI + rr;
      int dm, dn;
      G::piece_of(lane, i, t, dm, dn);
      const int m = m_base + dm, n = n_base + dn;
      f32x4_t lo = *reinterpret_cast<const f32x4_t*>(reg + row * ROWB + cc * 4);
      f32x4_t hi = *reinterpret_cast<const f32x4_t*>(reg + row * ROWB + cc * 4 + 16);
      if (GUARD && (m >= p.M || n >= p.N)) continue;
      lo *= alpha;
      hi *= alpha;
      if (use_c) {
        const uint32_t w[4] = {cin[i % CW][t].x, cin[i % CW][t].y, cin[i % CW][t].z, cin[i % CW][t].w};
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
        lo *= p.out_scale;
        hi *= p.out_scale;
        if constexpr (!GUARD) {
          if (p.out_transposed) {
            *reinterpret_cast<f32x4_t*>(reg + row * ROWB + cc * 4) = lo;
            *reinterpret_cast<f32x4_t*>(reg + row * ROWB + cc * 4 + 16) = hi;
            continue;
          }
        }
        if constexpr (RMW) {  // in-place update of a float32 matrix (optimizer step folded into the epilogue)
          const f32x4_t olo = oldv[i % OW][2 * t], ohi = oldv[i % OW][2 * t + 1];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            lo[e] = __builtin_fmaf(p.out_accum, olo[e], lo[e]);
            hi[e] = __builtin_fmaf(p.out_accum, ohi[e], hi[e]);
          }
        }
        *reinterpret_cast<f32x4_t*>(o) = lo;
        *reinterpret_cast<f32x4_t*>(o + 4) = hi;
      } else {
        uint16_t* o = reinterpret_cast<uint16_t*>(p.Out) + batch * p.o_bs + (int64_t)m * p.ldo + n;
        const uint2 a = __builtin_bit_cast(uint2, __builtin_convertvector(lo, bf16x4_t));
        const uint2 b = __builtin_bit_cast(uint2, __builtin_convertvector(hi, bf16x4_t));
        *reinterpret_cast<uint4*>(o) = make_uint4(a.x, a.y, b.x, b.y);
      }
    }
    if constexpr (OUT_F32 && !GUARD && MI == 16) {
      if (p.out_transposed) {
        const int col = lane & 15, g4 = 4 * (lane >> 4);
#pragma unroll
        for (int t = 0; t < TN / 16; ++t) {
          f32x4_t w;
#pragma unroll
          for (int e = 0; e < 4; ++e) w[e] = *reinterpret_cast<const float*>(reg + (g4 + e) * ROWB + (16 * t + col) * 4);
          int dm, dn;
          G::transposed_piece_of(lane, i, t, dm, dn);
          float* o = reinterpret_cast<float*>(p.Out) + batch * p.o_bs + (int64_t)(n_base + dn) * p.ldo + m_base + dm;
          if constexpr (RMW) {
            const f32x4_t old = oldv[i % OW][t];
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = __builtin_fmaf(p.out_accum, old[e], w[e]);
          }
          *reinterpret_cast<f32x4_t*>(o) = w;
        }
      }
    }
    // this block's registers take the pieces of a later block
    if (i + CW < C::FM) load_cin(i + CW);
    if (RMW && i + OW < C::FM) load_old(i + OW);
  }
  if (p.slots_out != nullptr) {
    const float total = block_sum_f32<C::NT>(ssq, red);
    if (threadIdx.x == 0) p.slots_out[batch * p.slot_stride + p.slot_base + blockIdx.x] = total;
  }
}

// SYRK-mode epilogue through LDS.  The accumulator layout gives a lane one output row and 4-column groups, i.e.
// 8-byte pieces of 16 different rows per store instruction, and the mirrored tile would go out as single bf16
// values.  Here the finished bf16 tile is assembled in LDS (row-major, rows padded by 16 bytes) and written
// with 16 bytes per lane along rows; the mirror image is formed from the same staged rows with the LDS transpose
// read (4 x 4 blocks of bf16 transposed in flight) and also leaves with 16 bytes per lane along (mirrored) rows.
// A diagonal tile is made symmetric in LDS first: the wavefronts on the diagonal stage the lower half of their
// block and fill its upper half with transposed 4 x 4 blocks; the block below the diagonal is written like any
// other and mirrored into the tile's upper right.  The stored result is therefore symmetric bit for bit.
// The staging area may be larger than the ring (a 256 x 256 tile: 132 KB against 128 KB); the kernel sizes its LDS
// for the larger of the two.
// The addends (the beta terms) reach the accumulators in one of two ways.  Tiles of up to 192 x 192 read them straight
// in accumulator layout (8 bytes per quad, whole 32-byte sectors per row), the first one before the K loop, the second
// at the start of the epilogue.  A 256 x 256 tile has no registers to spare for that (256 accumulators per lane): its
// addend tiles are copied to the staging area by the whole workgroup with 16-byte row-wise loads and picked up from
// there in accumulator layout, one after the other; the finished values then overwrite them in place.
// Every wavefront of the workgroup must call this (it contains barriers).
// Geometry of the staged SYRK epilogue.
template <class C>
struct SyrkStage {
  static constexpr int TILE = C::TILE_M, LDT = TILE + 8;  // LDS row pitch in elements
  static constexpr int STAGE_BYTES = TILE * LDT * 2;
  static constexpr int CPRW = TILE / 8;              // 16-byte chunks per tile row
  static constexpr int NCH = TILE * CPRW / C::NT;    // chunks per thread
  // one 8-byte quad of an addend per accumulator quad: NQUAD x 2 registers per lane when held in registers
  static constexpr int NQUAD = C::FM * C::FN;
  static constexpr bool CIN_EARLY = NQUAD * 2 <= 80;
  static_assert(STAGE_BYTES <= 160 * 1024 - 256, "staging area exceeds the LDS");
  // Row-wise passes over the staged tile (the addend copy of the 256 x 256 tile, the write-out): piece u of thread tid
  // is the 16-byte chunk c8 of tile row `row`.
  static MI_HD void chunk_of(int tid, int u, int& row, int& c8) {
    const int c = tid + u * C::NT;
    row = c / CPRW;
    c8 = c % CPRW;
  }
  // A diagonal tile holds nothing right of the diagonal block of a row (the wavefront that owns that block sits the
  // product out): that part comes from the mirror image, or stays unwritten when the upper triangle is skipped.
  static MI_HD bool chunk_held(bool diag, int row, int c8) { return !diag || c8 * 8 < (row / C::TM + 1) * C::TM; }
  // Mirrored write-out of staged rows [r_lo, r_lo + ROWS) x columns [0, CCOLS): a unit is 4 columns x 32 rows; each
  // 16-lane group transposes one unit with two LDS transpose reads (source lane L fetches the 4 columns at row
  // 8 (L % 4) + L / 4, then 4 rows further down) and ends up with 16 bytes of a mirrored row per lane.  For iteration
  // `it` of a lane: the staged element (src_row, src_col) its first read starts at, the row and first column of its
  // piece of the mirror image relative to that image's corner, and whether it stores at all.
  template <int ROWS, int CCOLS>
  static MI_HD bool mirror_piece(int it, int wave, int lane, int r_lo, int& src_row, int& src_col, int& drow, int& dcol) {
    static_assert(ROWS % 32 == 0 && CCOLS % 4 == 0, "units of 4 columns x 32 rows");
    constexpr int NB = ROWS / 32, UNITS = CCOLS / 4 * NB;
    const int l16 = lane & 15, unit = it * 16 + wave * 4 + (lane >> 4);
    const bool on = UNITS % 16 == 0 || unit < UNITS;
    const int u = (UNITS % 16 == 0 || unit < UNITS) ? unit : UNITS - 1;
    const int cq = u / NB, rb = u % NB;
    src_row = r_lo + 32 * rb + 8 * (l16 & 3) + (l16 >> 2);
    src_col = 4 * cq;
    drow = 4 * cq + (l16 & 3);
    dcol = 32 * rb + 8 * (l16 >> 2);
    return on;
  }
  template <int ROWS, int CCOLS>
  static constexpr int mirror_iterations() { return (CCOLS / 4 * (ROWS / 32) + 15) / 16; }
};
// This lane's addend values of a one-pass tile, in accumulator layout: quad (i, j) covers row
// m0 + mw + 16 i + (lane % 16), columns n0 + nw + 16 j + 4 (lane / 16) .. + 3.  One load
// instruction touches MI rows with 32 contiguous bytes each -- whole 32-byte sectors, so nothing is fetched twice.
// Issued before the K loop (first addend) or at the start of the epilogue (second), so that the burst of all
// workgroups does not sit on the critical path.
// Exactly NQUAD load instructions, whatever the position of the tile: the K loop that follows counts them in its
// vmcnt waits.  Quads beyond the matrix (GUARD) therefore read a clamped, valid address instead of being skipped; the
// values they deliver belong to outputs that are never stored.
// syrk_addend_elem: element offset (from the addend matrix of this batch entry) of the piece quad (i, j) of `lane` reads.
template <class C, bool GUARD>
MI_HD int64_t syrk_addend_elem(int M, int N, int64_t ldc, int lane, int m_base, int n_base, int i, int j) {
  constexpr int MI = C::MI;
  int m = m_base + i * MI + (lane & (MI - 1)), n = n_base + j * MI + 4 * (lane / MI);
  if constexpr (GUARD) {
    m = m < M ? m : M - 1;
    n = n + 4 <= N ? n : N - 4;
  }
  return (int64_t)m * ldc + n;
}
template <class C, bool GUARD>
__device__ __forceinline__ void syrk_addend_fetch(const GemmParams& p, const uint16_t* __restrict__ Cb, int lane, int m_base,
                                                  int n_base, uint2 (&pre)[SyrkStage<C>::NQUAD]) {
#pragma unroll
  for (int i = 0; i < C::FM; ++i)
#pragma unroll
    for (int j = 0; j < C::FN; ++j)
{
        pre[i * C::FN + j] = *reinterpret_cast<const uint2*>(Cb + syrk_addend_elem<C, GUARD>(p.M, p.N, p.ldc, lane, m_base, n_base, i, j));
      }
}

template <class C, bool GUARD>
__device__ __forceinline__ void syrk_epilogue_lds(const GemmParams& p, f32x4_t (&acc)[C::FM][C::FN],
                                                  char* lds, int lane, int wm, int wn, int m0, int n0, int64_t batch,
                                                  bool diag, float alpha, float beta, float beta2, float shift,
                                                  const uint2 (&cin_pre)[SyrkStage<C>::CIN_EARLY ? SyrkStage<C>::NQUAD : 1]) {
  using S = SyrkStage<C>;
  constexpr int LDT = S::LDT, MI = C::MI, FM = C::FM, FN = C::FN, TILE = S::TILE;
  constexpr int CPRW = S::CPRW, NCH = S::NCH;
  static_assert(C::TILE_M == C::TILE_N, "square tiles");
  static_assert(C::WGM == 2 && C::WGN == 2 && C::TM == C::TN, "2 x 2 wavefronts with square blocks: the diagonal blocks are (0,0) and (1,1)");
  static_assert(TILE * CPRW % C::NT == 0, "write-out must divide evenly");
  const int tid = threadIdx.x;
  const int frow = lane & (MI - 1), fk = lane / MI;
  const int mw = wm * C::TM, nw = wn * C::TN;           // this wavefront's block inside the tile
  uint16_t* __restrict__ ob = reinterpret_cast<uint16_t*>(p.Out) + batch * p.o_bs;
  const uint16_t* __restrict__ Cb = p.Cin ? p.Cin + batch * p.c_bs : nullptr;
  const bool use_c = beta != 0.0f && Cb != nullptr;
  const uint16_t* __restrict__ Cb2 = p.Cin2 ? p.Cin2 + batch * p.c_bs : nullptr;
  const bool use_c2 = beta2 != 0.0f && Cb2 != nullptr;
  // whether this wavefront's block holds anything that is stored (see idle_wave in the kernel)
  const bool active = (m0 + mw < p.M) && (n0 + nw < p.N) && !(diag && nw >= mw + C::TM);

  auto add = [&](f32x4_t& v, const uint2& raw, float coef) {
    v[0] = __builtin_fmaf(coef, __uint_as_float(raw.x << 16), v[0]);
    v[1] = __builtin_fmaf(coef, __uint_as_float(raw.x & 0xffff0000u), v[1]);
    v[2] = __builtin_fmaf(coef, __uint_as_float(raw.y << 16), v[2]);
    v[3] = __builtin_fmaf(coef, __uint_as_float(raw.y & 0xffff0000u), v[3]);
  };
  auto finish = [&](f32x4_t v, int ml, int nl) -> uint2 {  // the shift on the diagonal, then one rounding to bf16
    if (p.shift_mode == SHIFT_GRAM && diag) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (nl + r == ml) v[r] -= shift;
    }
    return __builtin_bit_cast(uint2, __builtin_convertvector(v, bf16x4_t));
  };

  // Finished bf16 quads of this lane, when they are few enough to be kept in registers.
  uint2 val[S::CIN_EARLY ? FM : 1][S::CIN_EARLY ? FN : 1];
  // ---- values: alpha * acc (+ beta * Cin) (+ beta2 * Cin2) (- shift on the diagonal), rounded to bf16 ----
  if constexpr (S::CIN_EARLY) {
    // Both addends arrive in accumulator layout: the first was requested before the K loop, the second is
    // requested now and consumed after the first.
    uint2 c2[S::NQUAD];
    if (use_c2) {
      syrk_addend_fetch<C, GUARD>(p, Cb2, lane, m0 + mw, n0 + nw, c2);
      // while those loads are on their way (a burst of all workgroups: 4 - 5 us), alpha and the first addend go into
      // the accumulators; the same operations in the same order as below, so the result does not change
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          f32x4_t v;
#pragma unroll
          for (int r = 0; r < 4; ++r) v[r] = alpha * acc[i][j][r];
          if (use_c) add(v, cin_pre[i * FN + j], beta);
          acc[i][j] = v;
        }
      asm volatile("" ::: "memory");  // (keeps the uses of c2 behind this block)
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          f32x4_t v = acc[i][j];
          add(v, c2[i * FN + j], beta2);
          val[i][j] = finish(v, mw + i * MI + frow, nw + j * MI + 4 * fk);
        }
    } else {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          const int ml = mw + i * MI + frow, nl = nw + j * MI + 4 * fk;
          f32x4_t v;
#pragma unroll
          for (int r = 0; r < 4; ++r) v[r] = alpha * acc[i][j][r];
          if (use_c) add(v, cin_pre[i * FN + j], beta);
          val[i][j] = finish(v, ml, nl);
        }
    }
    __syncthreads();  // every wavefront has left the K loop: the ring can be reused as staging space
  } else {
    // Large tile: every addend tile goes through the staging area.  The workgroup copies it there row by row (16 bytes
    // per lane, whole rows per 32 lanes), each lane adds its quads to its accumulators, and the next addend or the
    // finished values overwrite it.
    // All NCH 16-byte pieces of an addend tile are requested at once (in batches of eight with a wait after each, every
    // batch sat out a memory latency of its own: 7 us per addend and tile), the first addend before the accumulators
    // are scaled, the second as soon as the first has left its registers for the staging area, so that it is on its
    // way while the first is added.
    uint4 buf[NCH];
    auto request = [&](const uint16_t* __restrict__ src) {
#pragma unroll
      for (int u = 0; u < NCH; ++u) {
        int row, c8;
        S::chunk_of(tid, u, row, c8);
        const int gr = m0 + row, gc = n0 + c8 * 8;
        buf[u] = make_uint4(0u, 0u, 0u, 0u);
        if (!GUARD || (gr < p.M && gc < p.N)) buf[u] = *reinterpret_cast<const uint4*>(src + (int64_t)gr * p.ldc + gc);
      }
    };
    auto park = [&]() {  // registers -> staging area (behind a barrier: nobody reads the area any more)
      __syncthreads();
#pragma unroll
      for (int u = 0; u < NCH; ++u) {
        int row, c8;
        S::chunk_of(tid, u, row, c8);
        *reinterpret_cast<uint4*>(lds + (row * LDT + c8 * 8) * 2) = buf[u];
      }
    };
    auto add_staged = [&](float coef) {
      __syncthreads();
      if (active) {
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
          for (int j = 0; j < FN; ++j) {
            const int ml = mw + i * MI + frow, nl = nw + j * MI + 4 * fk;
            add(acc[i][j], *reinterpret_cast<const uint2*>(lds + (ml * LDT + nl) * 2), coef);
          }
      }
    };
    if (use_c) request(Cb);
    else if (use_c2) request(Cb2);
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][j][r] *= alpha;
    if (use_c) {
      park();
      if (use_c2) request(Cb2);
      add_staged(beta);
    }
    if (use_c2) {
      park();
      add_staged(beta2);
    }
    __syncthreads();  // the area is free for the finished values
  }
  // finished bf16 quad (i, j) of this lane
  auto quad = [&](int i, int j) -> uint2 {
    if constexpr (S::CIN_EARLY)
      return val[i][j];
    else
      return finish(acc[i][j], mw + i * MI + frow, nw + j * MI + 4 * fk);
  };
  auto elem = [&](const uint2& q, int r) -> uint16_t {
    return (uint16_t)(r == 0 ? (q.x & 0xffffu) : r == 1 ? (q.x >> 16) : r == 2 ? (q.y & 0xffffu) : (q.y >> 16));
  };
  typedef s16x4_t __attribute__((address_space(3))) * lds_tr_ptr;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)lds;  // LDS byte address
  auto tr_read = [&](uint32_t byte_off) -> uint2 {
    return __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(uintptr_t)(lds_base + byte_off)));
  };
  const bool sym = diag && !p.skip_upper;  // diagonal tile: the lower half and its mirror image make the tile
  const int wave = tid >> 6, l16 = lane & 15;
  // Transposed write-out of staged rows [r_lo, r_lo + ROWS) x columns [0, CCOLS) to the image whose corner is
  // (grow0, gcol0); the geometry is SyrkStage::mirror_piece.
  auto mirror_out = [&](auto rows_c, auto ccols_c, int r_lo, int grow0, int gcol0) {
    constexpr int ROWS = decltype(rows_c)::value, CCOLS = decltype(ccols_c)::value;
    constexpr int ITER = S::template mirror_iterations<ROWS, CCOLS>();
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      int src_row, src_col, drow, dcol;
      const bool on = S::template mirror_piece<ROWS, CCOLS>(it, wave, lane, r_lo, src_row, src_col, drow, dcol);
      const uint32_t a0 = (uint32_t)((src_row * LDT + src_col) * 2);
      const uint2 t0 = tr_read(a0), t1 = tr_read(a0 + 4 * LDT * 2);
      const int gr = grow0 + drow, gc = gcol0 + dcol;
      if (on && (!GUARD || (gr < p.N && gc < p.M)))
        store16_through(ob + (int64_t)gr * p.ldo + gc, make_uint4(t0.x, t0.y, t1.x, t1.y));
    }
  };
  // ---- the tile, row-major ----
  if (!sym || wm > wn) {
#pragma unroll
    for (int i = 0; i < FM; ++i) {
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        const int ml = mw + i * MI + frow, nl = nw + j * MI + 4 * fk;
        *reinterpret_cast<uint2*>(lds + (ml * LDT + nl) * 2) = quad(i, j);
      }
    }
  } else if (wm == wn) {
    // block on the diagonal: quads below the diagonal's 4 x 4 blocks go in whole, a quad inside such a block
    // puts its lower elements at both positions; the rest of the upper half is filled in below
#pragma unroll
    for (int i = 0; i < FM; ++i) {
#pragma unroll
      for (int j = 0; j <= i; ++j) {
        const int ml = mw + i * MI + frow, nl = nw + j * MI + 4 * fk;
        if (j < i || nl < (ml & ~3)) {
          *reinterpret_cast<uint2*>(lds + (ml * LDT + nl) * 2) = quad(i, j);
        } else if (nl == (ml & ~3)) {
          const uint2 q4 = quad(i, j);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const uint16_t e = elem(q4, r);
            if (nl + r <= ml) *reinterpret_cast<uint16_t*>(lds + (ml * LDT + nl + r) * 2) = e;
            if (nl + r < ml) *reinterpret_cast<uint16_t*>(lds + ((nl + r) * LDT + ml) * 2) = e;
          }
        }
      }
    }
  }
  if (sym) {
    __syncthreads();
    if (wm == wn) {
      // upper 4 x 4 blocks of the diagonal block <- transposed lower ones (16 blocks per transpose read)
      constexpr int NB4 = C::TM / 4;
      static_assert(NB4 * NB4 % 16 == 0, "blocks must fill whole transpose reads");
      const int rowbase = mw, colbase = nw;
      for (int it = 0; it < NB4 * NB4 / 16; ++it) {
        const int ids = it * 16 + 4 * (lane >> 4) + (lane & 3);  // block this lane fetches a row of
        const uint2 t =
            tr_read((uint32_t)(((rowbase + 4 * (ids / NB4) + (l16 >> 2)) * LDT + colbase + 4 * (ids % NB4)) * 2));
        const int idr = it * 16 + (lane >> 2), br = idr / NB4, bc = idr % NB4;  // block this lane receives a column of
        if (br > bc) *reinterpret_cast<uint2*>(lds + ((rowbase + 4 * bc + (lane & 3)) * LDT + colbase + 4 * br) * 2) = t;
      }
    }
  }
  __syncthreads();
  // ---- row-wise write-out: LDS row -> global row m0 + row ----
#pragma unroll
  for (int it = 0; it < NCH; ++it) {
    int row, c8;
    S::chunk_of(tid, it, row, c8);
    const int gr = m0 + row, gc = n0 + c8 * 8;
    const uint4 v = *reinterpret_cast<const uint4*>(lds + (row * LDT + c8 * 8) * 2);
    const bool held = S::chunk_held(diag, row, c8);
    if (held && (!GUARD || (gr < p.M && gc < p.N))) store16_through(ob + (int64_t)gr * p.ldo + gc, v);
  }
  // ---- the mirror image, straight from the staged rows ----
  if (!p.skip_upper) {
    if (!diag) {
      mirror_out(std::integral_constant<int, TILE>{}, std::integral_constant<int, TILE>{}, 0, n0, m0);
    } else {
      // the block below the diagonal blocks (rows from TM on, columns before TM) goes to the upper right of the tile
      mirror_out(std::integral_constant<int, C::TM>{}, std::integral_constant<int, C::TM>{}, C::TM, n0, m0 + C::TM);
    }
  }
}

// s_waitcnt immediate for gfx9: vmcnt in bits [3:0] and [15:14], expcnt [6:4] = 7 (no wait), lgkmcnt [11:8].
constexpr int waitcnt_imm(int vmcnt, int lgkmcnt) {
  return (vmcnt & 15) | ((vmcnt >> 4) << 14) | 0x70 | ((lgkmcnt & 15) << 8);
}

// Lower-triangle launches number their tiles through the whole batch on a one-dimensional grid (GemmParams::lin_*):
// consecutive workgroup ids go round-robin to the 8 XCDs, so within a round of lin_g workgroups XCD x takes the
// lin_g / 8 consecutive tiles from x lin_g / 8 on, and of the `rest` tiles of the last, partial round the tiles
// [rest x / 8, rest (x + 1) / 8): the workgroups that share an L2 work on neighbouring tiles of (mostly) one
// matrix, and every XCD gets the same number of tiles, give or take one, whatever the tile count of one matrix is.
//
// STREAMK != 0: the two extra launches of a split-tail product (lower-triangle products of K-contiguous operands
// whose tiles do not fill whole rounds of the chip; 256 x 256 tiles).  The whole rounds, tiles [0, lin_tiles), go out
// as an ordinary launch.  Then
//   SK_PARTS   the sk_rem tiles left over, fewer than half a round, are split along K between sk_splits >= 2
//              workgroups each (XCD x takes the left-over tiles [x sk_tpx, (x + 1) sk_tpx)); a workgroup multiplies
//              its part of the K range and parks its float32 accumulators in global memory (accumulator layout of
//              the 256 x 256 tile, lane-linear), nothing else.
//   SK_FINISH  a kernel of 128 x 128 tiles without a K loop: four workgroups per left-over tile, one per 128 x 128
//              quarter (what one wavefront of SK_PARTS accumulated), add the parked accumulators in split order
//              and run the ordinary epilogue of a 128 x 128 tile.
// The launches follow each other on one stream; no workgroup ever waits for another one.  (Separate kernels and not
// one with several roles: a 256 x 256 tile leaves no register to spare, and a kernel that spills to scratch memory
// was measured 40 % slower on whole tiles.)
// Workgroup -> tile of an ordinary lower-triangle launch (the numbering described above); -1 for the workgroups that
// pad the last round to a multiple of 8.
MI_HD int tri_tile_of_block(int bid, int lin_tiles, int g) {
  const int full = lin_tiles / g * g;
  if (bid < full) return bid / g * g + (bid % 8) * (g / 8) + (bid % g) / 8;
  const int j = bid - full, rest = lin_tiles - full, lo = rest * (j % 8) / 8, hi = rest * (j % 8 + 1) / 8;
  if (j / 8 >= hi - lo) return -1;
  return full + lo + j / 8;
}
// SK_PARTS: workgroup -> (left-over tile, split, its K tiles [k_first, k_first + nk)); false for a padding workgroup.
MI_HD bool sk_part_of_block(int bid, int sk_tpx, int sk_rem, int sk_splits, int nk_full, int& sk_tile, int& sk_split,
                            int& k_first, int& nk) {
  sk_tile = (bid % 8) * sk_tpx + (bid / 8) % sk_tpx;
  sk_split = (bid / 8) / sk_tpx;
  if (sk_tile >= sk_rem || sk_split >= sk_splits) return false;
  k_first = nk_full * sk_split / sk_splits;
  nk = nk_full * (sk_split + 1) / sk_splits - k_first;
  return true;
}
// SK_FINISH: workgroup -> (left-over tile, quarter); the quarter is row half + 2 * column half = the wavefront of
// SK_PARTS that computed it.
MI_HD bool sk_quarter_of_block(int bid, int sk_rem, int& sk_tile, int& quarter) {
  sk_tile = bid / 4;
  quarter = bid % 4;
  return sk_tile < sk_rem;
}
constexpr int SK_TILE = 256, SK_NT = 256, SK_FN = 8;                       // the tile, threads and fragment columns of SK_PARTS
constexpr int64_t SK_IMAGE_FLOATS = (int64_t)SK_TILE * SK_TILE;            // one accumulator image
enum { SK_NONE = 0, SK_FINISH = 2, SK_PARTS = 3 };
// float4 index, in the array of accumulator images, of quad (i, j) of thread t (of the 256 x 256 tile's workgroup) in
// the image of split `split` of left-over tile `sk_tile`: image split sk_rem + sk_tile, quad (i SK_FN + j) SK_NT + t.
MI_HD int64_t sk_image_quad(int split, int sk_rem, int sk_tile, int i, int j, int t) {
  return ((int64_t)split * sk_rem + sk_tile) * (SK_IMAGE_FLOATS / 4) + (int64_t)(i * SK_FN + j) * SK_NT + t;
}
// RMW: GEMM mode with float32 output only, the variant that launch_fast takes for p.out_accum != 0 (see
// gemm_epilogue_lds).
template <class C, bool P_KS, bool Q_KS, int MODE, bool OUT_F32, bool EDGE, int STREAMK = 0, bool RMW = false>
__global__ void __launch_bounds__(C::NT) gemm_fast_kernel(GemmParams p) {
  constexpr int NS = C::NS, FM = C::FM, FN = C::FN, P_BYTES = C::P_BYTES, NT = C::NT;
  // The ring of operand slots; every LDS access of the K loop names its slot statically (ring[u] is a constant
  // offset into one LDS array).  The lower-triangle epilogue reuses the memory as its staging area, which may be
  // larger than the ring, so the array is sized for the larger of the two.
  constexpr bool SYRK_STAGED = MODE == MODE_SYRK && !OUT_F32 && C::NW == 4;
  constexpr int RING_BYTES = NS * C::SLOT_BYTES;
  constexpr int LDS_BYTES = (SYRK_STAGED && SyrkStage<C>::STAGE_BYTES > RING_BYTES) ? SyrkStage<C>::STAGE_BYTES : RING_BYTES;
  __shared__ __align__(1024) char lds_mem[LDS_BYTES];
  char(*const ring)[C::SLOT_BYTES] = reinterpret_cast<char(*)[C::SLOT_BYTES]>(lds_mem);
  __shared__ float red[NT / 64];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: everything derived from it stays in SGPRs
  const int wm = wave % C::WGM, wn = wave / C::WGM;
  static_assert(!RMW || (MODE == MODE_GEMM && OUT_F32 && !EDGE && (C::TN == 32 || C::TN == 64 || C::TN == 128)), "in-place variant: staged GEMM epilogue");
  static_assert(!STREAMK || (MODE == MODE_SYRK && !P_KS && !Q_KS && !EDGE && !OUT_F32 && C::NW == 4), "stream-K variant");
  static_assert(!STREAMK || (STREAMK == SK_FINISH ? (C::TILE_M == 128 && C::WGM == 2) : (C::TILE_M == SK_TILE && C::NT == SK_NT && C::FN == SK_FN)),
                "SK_PARTS on 256 x 256 tiles, SK_FINISH on their 128 x 128 quarters");
  int64_t batch = blockIdx.y;
  int tm, tn;
  int k_first = 0, nk = p.K / C::BK;  // K tiles of this pass: [k_first, k_first + nk)
  int sk_tile = 0, sk_split = 0;  // left-over tile and K split of this workgroup (SK_PARTS); tile and quarter (SK_FINISH)
  if constexpr (MODE == MODE_SYRK) {
    const int tri = p.tiles_m * (p.tiles_m + 1) / 2, bid = (int)blockIdx.x;
    int tile;
    if constexpr (STREAMK == SK_NONE) {
      tile = tri_tile_of_block(bid, p.lin_tiles, p.lin_g);
      if (tile < 0) return;  // padding workgroup (leaves before any barrier)
    } else {
      if constexpr (STREAMK == SK_PARTS) {
        if (!sk_part_of_block(bid, p.sk_tpx, p.sk_rem, p.sk_splits, p.K / C::BK, sk_tile, sk_split, k_first, nk)) return;  // padding workgroup
      } else {
        if (!sk_quarter_of_block(bid, p.sk_rem, sk_tile, sk_split)) return;
      }
      tile = p.lin_tiles + sk_tile;
    }
    batch = tile / tri;
    tri_block_decode(tile % tri, p.tiles_m, tm, tn);  // (for SK_FINISH, p.tiles_m counts 256 x 256 tiles)
    if constexpr (STREAMK == SK_FINISH) {
      const int qm = sk_split % 2, qn = sk_split / 2;
      if (tm == tn && qn > qm) return;  // the quarter above the diagonal of a diagonal tile: written as a mirror image
      tm = 2 * tm + qm;
      tn = 2 * tn + qn;
    }
  } else {
    gemm_tile_of((int)blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
  }
  const int m0 = tm * C::TILE_M, n0 = tn * C::TILE_N;

  FastLoader<C, P_KS, C::TILE_M, EDGE> lp;
  FastLoader<C, Q_KS, C::TILE_N, EDGE> lq;
  int64_t p_off = batch * p.p_bs, q_off = batch * p.q_bs;
  if (p.batch_inner > 1) {  // K slices of one matrix as separate batch entries (split-K products)
    const int64_t outer = batch / p.batch_inner, inner = batch % p.batch_inner;
    p_off = outer * p.p_bs + inner * p.p_bs2;
    q_off = outer * p.q_bs + inner * p.q_bs2;
  }
  // A wavefront none of whose outputs is ever stored (its rows or columns lie beyond the matrix, or its block is
  // strictly above the diagonal of a diagonal SYRK tile) keeps loading its share of the operand tiles and keeps
  // every barrier, but issues no fragment reads and no MFMAs: on this part the clock follows the power drawn,
  // so work that is thrown away slows down the work that is kept.
  const bool idle_wave = (m0 + wm * C::TM >= p.M) || (n0 + wn * C::TN >= p.N) ||
                         (MODE == MODE_SYRK && tm == tn && wn * C::TN >= (wm + 1) * C::TM);

  constexpr int MI = C::MI, ACC_N = 4;
  f32x4_t acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int e = 0; e < ACC_N; ++e) acc[i][j][e] = 0.0f;

  constexpr int NQ = C::BK / C::KI;  // k-steps of one tile
  constexpr int LOADS_PER_TILE = C::LPT_P + C::LPT_Q;  // per thread, both operands
  static_assert(NQ % 2 == 0, "fragment buffer parity assumes an even number of k-steps per tile");
  static_assert((NS - 1) * LOADS_PER_TILE < 64, "vmcnt is a 6-bit counter");

  // Pipeline.  Ring slot kt % NS holds K tile kt; while tile kt is multiplied, tiles kt+1 .. kt+NS-1 are in
  // flight.  Per tile: k-steps 0 .. NQ-2 (each fetches the fragments of the next k-step into the other
  // register buffer), then wait for this wavefront's loads of tile kt+1 and its own LDS reads, one barrier
  // (tile kt+1 is published; nobody reads slot kt % NS any more), then the last k-step, which also fetches
  // the first fragments of tile kt+1 and starts the loads of tile kt+NS into the slot just vacated.
  // Every k-step is written as MFMA "slots": one MFMA followed by its share of the LDS reads and of the
  // direct-to-LDS loads, pinned in that order, so that a wavefront that has the SIMD to itself never stops
  // issuing MFMAs while it feeds the memory pipes.
  // The loads of a tile are cut into PARTS equal parts.  With three or more ring slots the parts go out one
  // per k-step (part 0 right after the barrier that vacates the slot, the rest in the k-steps of the next
  // tile before its barrier): the CU's single address unit then sees an even stream instead of a burst from
  // all wavefronts at once, and the tile still has NS-2 whole tile times to land.  With two slots there is no
  // slack for that and the whole tile goes out in the k-step after the barrier.
  constexpr int UNITS = FM + FN, MMAS = FM * FN;  // fragment reads / MFMAs per k-step
  constexpr int UPS = (UNITS + MMAS - 1) / MMAS;  // fragment reads per slot
  constexpr int PARTS = (NS >= 3 && LOADS_PER_TILE % NQ == 0) ? NQ : 1;
  constexpr int PL = LOADS_PER_TILE / PARTS;      // loads per part
  constexpr int DPS = (PL + MMAS - 1) / MMAS;     // loads per slot (1 unless a part outnumbers the MFMAs)
  bf16x8_t fp[2][FM], fq[2][FN];
  uint32_t ks_sp = 0, ks_rp = 0, ks_sq = 0, ks_rq = 0;  // lane constants of the K-strided reads
  if constexpr (P_KS) ks16_consts<C::TILE_M>(lane, wm * C::TM, ks_sp, ks_rp);
  if constexpr (Q_KS) ks16_consts<C::TILE_N>(lane, wn * C::TN, ks_sq, ks_rq);
  auto lds_of = [&](const char* ptr) { return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)ptr; };
  auto read_unit = [&](const char* st, int q, int buf, int r) {
    if (r < FM) {
      if constexpr (P_KS)
        fp[buf][r] = fast_frag16_ks<C::TILE_M>(lds_of(st), ks_sp, ks_rp, r, q);
      else
        fp[buf][r] = fast_frag<C>(st, wm * C::TM + r * MI, q, lane);
    } else {
      if constexpr (Q_KS)
        fq[buf][r - FM] = fast_frag16_ks<C::TILE_N>(lds_of(st + P_BYTES), ks_sq, ks_rq, r - FM, q);
      else
        fq[buf][r - FM] = fast_frag<C>(st + P_BYTES, wn * C::TN + (r - FM) * MI, q, lane);
    }
  };
  auto fetch = [&](const char* st, int q, int buf) {
#pragma unroll
    for (int r = 0; r < UNITS; ++r) read_unit(st, q, buf, r);
  };
  const uint32_t ring_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)&ring[0][0];
  auto issue_one = [&](int slot, int d) {  // d-th load of this wavefront for a tile: P blocks first, then Q
    if (d < C::LPT_P)
      lp.issue_one(ring_lds + slot * C::SLOT_BYTES, wave, d);
    else
      lq.issue_one(ring_lds + slot * C::SLOT_BYTES + P_BYTES, wave, d - C::LPT_P);
  };
  // parts [p0, p1) of the current tile of the loaders in one go; the loaders move on after the last part
  auto issue_parts = [&](int slot, int p0, int p1) {
#pragma unroll
    for (int d = p0 * PL; d < p1 * PL; ++d) issue_one(slot, d);
    if (p1 == PARTS) {
      lp.advance();
      lq.advance();
    }
  };
  // One k-step on register buffer `buf`.  READ: fetch the fragments of k-step rd_q of tile rd_tile into the
  // other buffer.  PART >= 0: issue that part of the loaders' current tile into slot ld_slot.
  auto k_step = [&](auto read_flag, auto part, int buf, const char* rd_tile, int rd_q, int ld_slot) {
    constexpr bool READ = decltype(read_flag)::value;
    constexpr int PART = decltype(part)::value;
    if constexpr (P_KS || Q_KS) {
      // keep the address arithmetic of the transpose reads next to them (it would otherwise be hoisted out of
      // the K loop, one register per read)
      asm volatile("" : "+v"(ks_sp), "+v"(ks_rp), "+v"(ks_sq), "+v"(ks_rq));
    }
    static_for<MMAS>([&](auto xc) {
      // P fragment i stays for FN MFMAs in a row; the Q fragments are walked forth and back, so that one of the
      // two operands is always the same as in the previous MFMA (measurably less power than changing both)
      constexpr int x = decltype(xc)::value, i = x / FN, j = (i & 1) ? FN - 1 - x % FN : x % FN;
      mfma16_inplace(acc[i][j], fq[buf][j], fp[buf][i]);
      if constexpr (READ) {
        static_for<UPS>([&](auto uc) {
          constexpr int u = decltype(uc)::value;
          if constexpr (x * UPS + u < UNITS) read_unit(rd_tile, rd_q, buf ^ 1, x * UPS + u);
        });
      }
      if constexpr (PART >= 0) {
        // load e of the part goes into slot e * MMAS / PL when the part has fewer loads than the k-step has
        // MFMAs (an even spread), else DPS loads per slot
        static_for<PL>([&](auto ec) {
          constexpr int e = decltype(ec)::value;
          if constexpr ((PL <= MMAS ? e * MMAS / PL : e / DPS) == x) issue_one(ld_slot, PART * PL + e);
        });
      }
      __builtin_amdgcn_sched_barrier(0);
    });
    if (PART == PARTS - 1) {
      lp.advance();
      lq.advance();
    }
  };
  // `steady` (a compile-time flag) marks tiles in the middle of the K loop: tile kt+NS exists (so the vacated
  // slot is refilled and NS-2 younger tiles stay in flight at the wait), and the tile body is branch free.
  // `extra` (compile time) and `with_extra` (run time, uniform): register loads issued between this wavefront's loads
  // of tile kt+1 and the wait below (the addend fetch in front of tile 0) that the wait must not sit out.
  auto k_tile = [&](auto steady, int kt, int cur_slot, const char* cur, const char* nxt, auto extra, bool with_extra) {
    constexpr bool STEADY = decltype(steady)::value;
    constexpr int EXTRA = decltype(extra)::value;
    static_assert((NS - 2) * LOADS_PER_TILE + EXTRA < 64, "vmcnt is a 6-bit counter");
    const int prev_slot = (cur_slot + NS - 1) % NS;  // receives the later parts of tile kt-1+NS
    if (!STEADY && PARTS > 1 && kt + NS - 1 < nk) issue_parts(prev_slot, 1, PARTS);
#pragma unroll
    for (int q = 0; q + 1 < NQ; ++q) {
      if (STEADY && PARTS > 1) {
        if (q == 0) k_step(std::true_type{}, std::integral_constant<int, (PARTS > 1 ? 1 : -1)>{}, q & 1, cur, q + 1, prev_slot);
        if (q == 1) k_step(std::true_type{}, std::integral_constant<int, (PARTS > 2 ? 2 : -1)>{}, q & 1, cur, q + 1, prev_slot);
        if (q == 2) k_step(std::true_type{}, std::integral_constant<int, (PARTS > 3 ? 3 : -1)>{}, q & 1, cur, q + 1, prev_slot);
      } else {
        k_step(std::true_type{}, std::integral_constant<int, -1>{}, q & 1, cur, q + 1, 0);
      }
    }
    // own loads of tile kt+1 have landed; own reads of `cur` are done
    if (STEADY && EXTRA > 0 && with_extra)
      __builtin_amdgcn_s_waitcnt(waitcnt_imm((NS - 2) * LOADS_PER_TILE + EXTRA, 0));
    else
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(STEADY ? (NS - 2) * LOADS_PER_TILE : 0, 0));
    __syncthreads();
    if (STEADY) {
      k_step(std::true_type{}, std::integral_constant<int, 0>{}, (NQ - 1) & 1, nxt, 0, cur_slot);
    } else {
      if (kt + NS < nk) issue_parts(cur_slot, 0, 1);
      if (kt + 1 < nk) fetch(nxt, 0, 0);
      k_step(std::false_type{}, std::integral_constant<int, -1>{}, (NQ - 1) & 1, nxt, 0, 0);
    }
  };
  static_assert(NQ <= 4, "k_tile spells out at most three k-steps before the barrier");

  constexpr bool CIN_EARLY = SYRK_STAGED && SyrkStage<C>::CIN_EARLY;
  uint2 cin_pre[CIN_EARLY ? SyrkStage<C>::NQUAD : 1];
  if constexpr (STREAMK != SK_FINISH) {
    lp.init(p.P + p_off + (STREAMK ? (int64_t)k_first * C::BK : 0), p.ldp, m0, p.M, wave, lane);
    lq.init(p.Q + q_off + (STREAMK ? (int64_t)k_first * C::BK : 0), p.ldq, n0, p.N, wave, lane);
    // prologue: tiles 0 .. NS-2 and part 0 of tile NS-1 in flight, wait for tile 0
#pragma unroll
    for (int t = 0; t < NS - 1; ++t)
      if (t < nk) issue_parts(t, 0, PARTS);
    if (NS - 1 < nk) issue_parts(NS - 1, 0, 1);
    if (nk >= NS)
      __builtin_amdgcn_s_waitcnt(waitcnt_imm((NS - 2) * LOADS_PER_TILE + PL, 15));
    else
      __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));
    __syncthreads();
    // The first addend is requested here, behind the loads of the first tiles and in front of everything the K loop
    // issues.  The wait at the end of tile 0 (for tile 1, whose loads are older) lets these NQUAD loads stay in
    // flight: sat out there, the burst of all workgroups cost 4 us per launch.  From tile 1 on every wait is for loads
    // that are younger than the addend, so it has arrived by then whatever the count says.
    bool addend_in_flight = false;
    if constexpr (CIN_EARLY) {
      if (p.Cin != nullptr) {
        syrk_addend_fetch<C, EDGE>(p, p.Cin + batch * p.c_bs, lane, m0 + wm * C::TM, n0 + wn * C::TN, cin_pre);
        addend_in_flight = true;
      }
    }
    constexpr int ADDEND_LOADS = CIN_EARLY ? SyrkStage<C>::NQUAD : 0;
    if (idle_wave) {
      for (int kt = 0; kt < nk; ++kt) {
        const int cur_slot = kt % NS, prev_slot = (cur_slot + NS - 1) % NS;
        if (PARTS > 1 && kt + NS - 1 < nk) issue_parts(prev_slot, 1, PARTS);
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
        __syncthreads();
        if (kt + NS < nk) issue_parts(cur_slot, 0, 1);
      }
    } else {
      fetch(ring[0], 0, 0);
      int kt = 0;
      for (; kt + 2 * NS - 1 < nk; kt += NS) {  // every tile of this round is a steady one
        if constexpr (ADDEND_LOADS > 0) {
          k_tile(std::true_type{}, kt, 0, ring[0], ring[1 % NS], std::integral_constant<int, ADDEND_LOADS>{}, addend_in_flight && kt == 0);
#pragma unroll
          for (int u = 1; u < NS; ++u)
            k_tile(std::true_type{}, kt + u, u, ring[u], ring[(u + 1) % NS], std::integral_constant<int, 0>{}, false);
        } else {
#pragma unroll
          for (int u = 0; u < NS; ++u)
            k_tile(std::true_type{}, kt + u, u, ring[u], ring[(u + 1) % NS], std::integral_constant<int, 0>{}, false);
        }
      }
      for (; kt < nk; kt += NS) {
#pragma unroll
        for (int u = 0; u < NS; ++u)
          if (kt + u < nk) k_tile(std::false_type{}, kt + u, u, ring[u], ring[(u + 1) % NS], std::integral_constant<int, 0>{}, false);
      }
    }
    mfma_drain();
  }
  // Scalars, then the write-out of the finished accumulators.
  auto finish = [&]() __attribute__((always_inline)) {
    const Scalars sc = resolve_shift<NT>(p, batch, red, MODE == MODE_SYRK ? (tm == 0 && tn == 0) : blockIdx.x == 0);
    const float alpha = sc.alpha, beta = sc.beta, beta2 = sc.beta2, shift = sc.shift;
    const bool diag = (MODE == MODE_SYRK) && (tm == tn);
    if constexpr (MODE == MODE_GEMM && (C::TN == 32 || C::TN == 64 || C::TN == 128)) {
      __syncthreads();  // every wavefront has finished reading the ring: it can be reused as staging space
      gemm_epilogue_lds<C, OUT_F32, EDGE, RMW>(p, acc, &ring[0][0], wave, lane, m0 + wm * C::TM, n0 + wn * C::TN, batch, alpha,
                                               beta, red);
    } else if constexpr (SYRK_STAGED) {
      syrk_epilogue_lds<C, EDGE>(p, acc, &ring[0][0], lane, wm, wn, m0, n0, batch, diag, alpha, beta, beta2, shift, cin_pre);
    } else {
      tile_epilogue<MODE, OUT_F32, EDGE, FM, FN, NT, MI>(p, acc, m0 + wm * C::TM, n0 + wn * C::TN, lane, batch, diag, alpha, beta, shift,
                                                         red, beta2);
    }
  };
  if constexpr (STREAMK == SK_PARTS) {
    // image of split s of left-over tile t: slot s sk_rem + t; quad (i, j) of thread t at ((i SK_FN + j) SK_NT + t) float4s
    if (!idle_wave) {
      f32x4_t* img = reinterpret_cast<f32x4_t*>(p.sk_partials);
      static_for<FM>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
#pragma unroll
        for (int j = 0; j < FN; ++j) img[sk_image_quad(sk_split, p.sk_rem, sk_tile, i, j, tid)] = acc[i][j];
        __builtin_amdgcn_sched_barrier(0);  // one fragment row at a time: the image must not pile up in registers
      });
    }
    return;
  }
  if constexpr (STREAMK == SK_FINISH) {
    if constexpr (CIN_EARLY) {
      if (p.Cin != nullptr)
        syrk_addend_fetch<C, EDGE>(p, p.Cin + batch * p.c_bs, lane, m0 + wm * C::TM, n0 + wn * C::TN, cin_pre);
    }
    if (!idle_wave) {
      // this wavefront's 64 x 64 block inside the quarter = fragments (wm FM + i, wn FN + j) of wavefront sk_split of SK_PARTS
      const f32x4_t* img = reinterpret_cast<const f32x4_t*>(p.sk_partials);
      for (int s = 0; s < p.sk_splits; ++s) {
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
          for (int j = 0; j < FN; ++j) {
            const f32x4_t v = img[sk_image_quad(s, p.sk_rem, sk_tile, wm * FM + i, wn * FN + j, sk_split * 64 + lane)];
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][e] += v[e];
          }
      }
    }
  }
  finish();
}

}  // namespace mi
