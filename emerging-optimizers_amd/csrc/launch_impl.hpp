// Definitions of the launchers declared in launch.hpp; included by the translation units that instantiate kernels.
#pragma once
#include "../../include/mi_ns.h"
#include "launch.hpp"

namespace mi {

// Per-workgroup partial sums go to slots_out[batch * slot_stride + slot_base + workgroup]: refuse a launch whose
// workgroups would write past the capacity the caller reserved (checked before anything is launched).
static inline int check_slots(const GemmParams& q, int64_t tiles) {
  if (q.slots_out != nullptr && q.slot_capacity > 0 && (q.slot_base + tiles > q.slot_capacity || q.slot_stride > q.slot_capacity))
    return fail(MI_ERR_WORKSPACE, "internal: %lld partial-sum slots exceed the %d reserved", (long long)(q.slot_base + tiles),
                q.slot_capacity);
  return MI_OK;
}

template <int BM, int BN, int BK, int WGM, int WGN, bool P_KS, bool Q_KS, int MODE, bool OUT_F32>
int launch_one(const GemmParams& p, int64_t batch, hipStream_t stream) {
  auto kern = gemm_bf16_kernel<BM, BN, BK, WGM, WGN, P_KS, Q_KS, MODE, OUT_F32>;
  constexpr int LDS_BYTES = 2 * (BM + BN) * BK * 2;
  static bool attr_set = false;  // benign race: setting the attribute twice is harmless
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
    if (e != hipSuccess) return fail(MI_ERR_LAUNCH, "hipFuncSetAttribute(%d B LDS): %s", LDS_BYTES, hipGetErrorString(e));
    attr_set = true;
  }
  if (p.out_transposed) return fail(MI_ERR_UNSUPPORTED_SHAPE, "internal: the general kernel has no transposed output");
  GemmParams q = p;
  q.tiles_m = (p.M + BM - 1) / BM;
  q.tiles_n = (p.N + BN - 1) / BN;
  const int64_t tiles = (MODE == MODE_SYRK) ? (int64_t)q.tiles_m * (q.tiles_m + 1) / 2 : (int64_t)q.tiles_m * q.tiles_n;
  if (tiles <= 0 || batch <= 0) return MI_OK;
  if (batch > 65535) return fail(MI_ERR_UNSUPPORTED_SHAPE, "batch %lld exceeds the grid limit 65535", (long long)batch);
  if (q.slot_stride == 0) q.slot_stride = (int)tiles;
  if (int rc = check_slots(q, tiles)) return rc;
  g_last_launch = LastLaunch{(int)tiles, BM, BN, 0};
  dim3 grid((unsigned)tiles, (unsigned)batch, 1), block(WGM * WGN * 64, 1, 1);
#ifdef MI_HOST_CHECK
  host_check::general_launch(q, batch, P_KS, Q_KS, MODE == MODE_SYRK, OUT_F32, tiles);
#endif
  hipLaunchKernelGGL(kern, grid, block, LDS_BYTES, stream, q);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
  return MI_OK;
}

// Workgroups of configuration C that the chip holds at once, rounded down to a multiple of 8 (the XCDs): two per CU
// when two rings fit the LDS of a CU, else one.
template <class C>
int fast_round_size() {
  constexpr int per_cu = 2 * C::NS * C::SLOT_BYTES <= 160 * 1024 ? 2 : 1;
  const int g = device_cus() * per_cu / 8 * 8;
  return g >= 8 ? g : 8;
}

template <class C, bool P_KS, bool Q_KS, int MODE, bool OUT_F32>
int launch_fast(const GemmParams& p, int64_t batch, hipStream_t stream, int64_t tile_limit) {
  // the K loop of the fast kernel has no tail, and its loaders trust these extents
  if (p.K < C::BK || p.K % C::BK != 0)
    return fail(MI_ERR_UNSUPPORTED_SHAPE, "internal: K = %d is not a multiple of %d", p.K, C::BK);
  if (p.M <= 0 || p.N <= 0 || batch <= 0) return MI_OK;
  // transposed output: only the staged epilogue of the GEMM mode writes it, and only for whole tiles
  constexpr bool STAGED_GEMM = MODE == MODE_GEMM && OUT_F32 && C::MI == 16 && (C::TN == 32 || C::TN == 64 || C::TN == 128);
  if (p.out_transposed && !(STAGED_GEMM && p.M % C::TILE_M == 0 && p.N % C::TILE_N == 0 && p.ldo >= p.M && p.ldo % 4 == 0))
    return fail(MI_ERR_UNSUPPORTED_SHAPE, "internal: no transposed output for this product (%d x %d)", p.M, p.N);
  GemmParams q = p;
  q.tiles_m = (p.M + C::TILE_M - 1) / C::TILE_M;
  q.tiles_n = (p.N + C::TILE_N - 1) / C::TILE_N;
  dim3 grid;
  int64_t tiles;
  if constexpr (MODE == MODE_SYRK) {
    // one-dimensional grid over the tiles of the whole batch: whole rounds, then a last round with the same number
    // of tiles for every XCD
    tiles = (int64_t)q.tiles_m * (q.tiles_m + 1) / 2 * batch;
    if (tile_limit >= 0 && tile_limit < tiles) tiles = tile_limit;
    if (tiles > (int64_t)1 << 30) return fail(MI_ERR_UNSUPPORTED_SHAPE, "%lld tiles exceed the grid limit", (long long)tiles);
    if (tiles == 0) return MI_OK;
    q.lin_tiles = (int)tiles;
    q.lin_g = fast_round_size<C>();
    const int full = q.lin_tiles / q.lin_g * q.lin_g;
    grid = dim3((unsigned)(full + (q.lin_tiles - full + 7) / 8 * 8), 1, 1);
  } else {
    tiles = (int64_t)q.tiles_m * q.tiles_n;
    if (batch > 65535) return fail(MI_ERR_UNSUPPORTED_SHAPE, "batch %lld exceeds the grid limit 65535", (long long)batch);
    if (q.slot_stride == 0) q.slot_stride = (int)tiles;
    if (int rc = check_slots(q, tiles)) return rc;
    grid = dim3((unsigned)tiles, (unsigned)batch, 1);
  }
  const bool edge = (p.M % C::TILE_M) != 0 || (p.N % C::TILE_N) != 0;
  // (the loaders of an edge tile address its rows with 32-bit byte offsets from the tile's first row)
  if (edge && ((int64_t)C::TILE_M * p.ldp >= ((int64_t)1 << 31) || (int64_t)C::TILE_N * p.ldq >= ((int64_t)1 << 31)))
    return fail(MI_ERR_UNSUPPORTED_SHAPE, "internal: leading dimension too large for an edge tile");
  // Only the lower-triangle product of K-contiguous operands has a variant for tiles that overhang the matrix
  // (rows clamped in the loaders, guarded epilogue).
  constexpr bool HAS_EDGE_VARIANT = MODE == MODE_SYRK && !P_KS && !Q_KS;
  if (edge) {
    if constexpr (HAS_EDGE_VARIANT)
      MI_LAUNCH_FAST(C, P_KS, Q_KS, MODE, OUT_F32, true, 0, false, grid, stream, q);
    else
      return fail(MI_ERR_UNSUPPORTED_SHAPE, "internal: %d x %d is not a whole number of %d x %d tiles", p.M, p.N, C::TILE_M, C::TILE_N);
  } else {
    constexpr bool HAS_RMW_VARIANT = MODE == MODE_GEMM && OUT_F32 && (C::TN == 32 || C::TN == 64 || C::TN == 128);
    if constexpr (HAS_RMW_VARIANT) {
      if (p.out_accum != 0.0f)
        MI_LAUNCH_FAST(C, P_KS, Q_KS, MODE, OUT_F32, false, 0, true, grid, stream, q);
      else
        MI_LAUNCH_FAST(C, P_KS, Q_KS, MODE, OUT_F32, false, 0, false, grid, stream, q);
    } else {
      MI_LAUNCH_FAST(C, P_KS, Q_KS, MODE, OUT_F32, false, 0, false, grid, stream, q);
    }
  }
  g_last_launch = LastLaunch{(int)grid.x, C::TILE_M, C::TILE_N, 1};
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
  return MI_OK;
}

}  // namespace mi
