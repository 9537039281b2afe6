// Fast path of the bf16 tile engine for shapes that tile exactly (M % 256 == N % 256 == K % 64 == 0).
//
// 256 x 256 x 64 workgroup tile, 8 wavefronts (2 per SIMD) laid out 2 (M) x 4 (N), each owning a
// 128 x 64 sub-tile = 4 x 2 MFMA 32x32x16 accumulators (128 accumulator VGPRs).  Two wavefronts per
// SIMD let one issue MFMAs while the other waits on LDS or the barrier.
//
// Global -> LDS goes through the direct-to-LDS load (16 bytes per lane, a wavefront fills 1 KB of
// LDS at base + 16 * lane), two 64 KB stages, one barrier per K tile:
//     wait own loads of tile kt | barrier | issue loads of tile kt+1 into the other stage | MFMAs on tile kt
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

namespace fast {
constexpr int BM = 256, BN = 256, BK = 64;
constexpr int WGM = 2, WGN = 4, NW = WGM * WGN, NT = NW * 64;
constexpr int TM = BM / WGM, TN = BN / WGN, FM = TM / 32, FN = TN / 32;
constexpr int TILE_BYTES = 256 * BK * 2;  // one operand tile: 32 KB
constexpr int STAGE_BYTES = 2 * TILE_BYTES;
constexpr int LPT = TILE_BYTES / 1024 / NW;  // direct-to-LDS loads per wavefront per operand tile (4)
}  // namespace fast

__device__ __forceinline__ void dma16(const uint16_t* g, char* lds_wave_base) {
  __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)g,
                                   (void __attribute__((address_space(3)))*)lds_wave_base, 16, 0, 0);
}

// Per-thread global pointers of the direct-to-LDS loads of one operand tile.
template <bool KS>
struct FastLoader {
  const uint16_t* gp[fast::LPT];
  int64_t step;  // elements to advance per K tile

  __device__ __forceinline__ void init(const uint16_t* base, int64_t ld, int row0, int wave, int lane) {
#pragma unroll
    for (int i = 0; i < fast::LPT; ++i) {
      const int b = wave * fast::LPT + i;  // 1 KB block index inside the tile
      if (!KS) {
        const int row = 8 * b + (lane >> 3);
        const int c = (lane & 7) ^ ((row >> 1) & 7);
        gp[i] = base + (int64_t)(row0 + row) * ld + c * 8;
      } else {
        const int k = 2 * b + (lane >> 5);
        const int c = ((lane & 31) - 4 * k) & 31;
        gp[i] = base + (int64_t)k * ld + row0 + c * 8;
      }
    }
    step = KS ? (int64_t)fast::BK * ld : fast::BK;
  }
  __device__ __forceinline__ void issue(char* tile, int wave) {
#pragma unroll
    for (int i = 0; i < fast::LPT; ++i) {
      dma16(gp[i], tile + (wave * fast::LPT + i) * 1024);
      gp[i] += step;
    }
  }
};

// MFMA fragment (8 bf16 along k) for 32 consecutive rows starting at `row_base`, k-step q (16 k each).
template <bool KS>
__device__ __forceinline__ bf16x8_t fast_frag(const char* tile, int row_base, int q, int lane) {
  if (!KS) {
    const int row = row_base + (lane & 31);
    const int c = (2 * q + (lane >> 5)) ^ ((row >> 1) & 7);
    return *reinterpret_cast<const bf16x8_t*>(tile + row * 128 + c * 16);
  } else {
    const int i16 = lane & 15;
    const int col = row_base + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);
    const int kb = 16 * q + 8 * (lane >> 5) + (i16 >> 2);
    s16x4_t lo, hi;
    {
      const int k = kb;
      const int slot = ((col >> 3) + 4 * k) & 31;
      lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (s16x4_t __attribute__((address_space(3)))*)(tile + k * 512 + slot * 16 + (col & 7) * 2));
    }
    {
      const int k = kb + 4;
      const int slot = ((col >> 3) + 4 * k) & 31;
      hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (s16x4_t __attribute__((address_space(3)))*)(tile + k * 512 + slot * 16 + (col & 7) * 2));
    }
    typedef short s16x8_t __attribute__((ext_vector_type(8)));
    s16x8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8_t, both);
  }
}

template <bool P_KS, bool Q_KS, int MODE, bool OUT_F32>
__global__ void __launch_bounds__(fast::NT) gemm_fast_kernel(GemmParams p) {
  using namespace fast;
  __shared__ __align__(1024) char stage0[STAGE_BYTES];
  __shared__ __align__(1024) char stage1[STAGE_BYTES];
  __shared__ float red[NT / 64];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave % WGM, wn = wave / WGM;
  const int64_t batch = blockIdx.y;
  int tm, tn;
  if (MODE == MODE_SYRK) {
    tri_decode((int)blockIdx.x, tm, tn);
  } else {
    tm = (int)blockIdx.x % p.tiles_m;
    tn = (int)blockIdx.x / p.tiles_m;
  }
  const int m0 = tm * BM, n0 = tn * BN;

  FastLoader<P_KS> lp;
  FastLoader<Q_KS> lq;
  lp.init(p.P + batch * p.p_bs, p.ldp, m0, wave, lane);
  lq.init(p.Q + batch * p.q_bs, p.ldq, n0, wave, lane);

  f32x16_t acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  const int nk = p.K / BK;

  auto compute = [&](const char* st) {
#pragma unroll
    for (int q = 0; q < BK / 16; ++q) {
      bf16x8_t fp[FM], fq[FN];
#pragma unroll
      for (int i = 0; i < FM; ++i) fp[i] = fast_frag<P_KS>(st, wm * TM + i * 32, q, lane);
#pragma unroll
      for (int j = 0; j < FN; ++j) fq[j] = fast_frag<Q_KS>(st + TILE_BYTES, wn * TN + j * 32, q, lane);
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fq[j], fp[i], acc[i][j], 0, 0, 0);
    }
  };

  lp.issue(stage0, wave);
  lq.issue(stage0 + TILE_BYTES, wave);
  // Two K tiles per trip so that each stage is a distinct LDS object in every statement.
  for (int kt = 0; kt < nk; kt += 2) {
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wavefront's part of tile kt has landed
    __syncthreads();
    if (kt + 1 < nk) {
      lp.issue(stage1, wave);
      lq.issue(stage1 + TILE_BYTES, wave);
    }
    compute(stage0);
    if (kt + 1 < nk) {
      __builtin_amdgcn_s_waitcnt(0x0f70);
      __syncthreads();
      if (kt + 2 < nk) {
        lp.issue(stage0, wave);
        lq.issue(stage0 + TILE_BYTES, wave);
      }
      compute(stage1);
    }
  }

  float beta = p.beta;
  const float shift = resolve_shift<NT>(p, batch, red, beta);
  const bool diag = (MODE == MODE_SYRK) && (tm == tn);
  tile_epilogue<MODE, OUT_F32, false, FM, FN, NT>(p, acc, m0 + wm * TM, n0 + wn * TN, lane, batch, diag, p.alpha, beta,
                                                  shift, red);
}

}  // namespace mi
