// Lower-triangle fast kernels, K-contiguous operands: 256 x 256 and 128 x 128 (two-slot ring, two workgroups per CU) tiles.
#include "launch_impl.hpp"
namespace mi {
template int launch_fast<CfgBig, false, false, MODE_SYRK, false>(const GemmParams&, int64_t, hipStream_t, int64_t);
template int launch_fast<CfgT128x2, false, false, MODE_SYRK, false>(const GemmParams&, int64_t, hipStream_t, int64_t);

// ---- split-tail (stream-K) launch of the 256 x 256 tile ----
static constexpr size_t SK_IMAGE_BYTES = (size_t)SK_IMAGE_FLOATS * sizeof(float);  // 256 KB
static_assert(SK_IMAGE_FLOATS == (int64_t)CfgBig::NT * CfgBig::FM * CfgBig::FN * 4, "one float4 per thread and fragment");

StreamKPlan streamk_plan(int64_t tiles, int k_tiles, int cus) {
  StreamKPlan s{};
  s.rounds = (int)(tiles / cus);
  s.rem = (int)(tiles % cus);
  s.splits = 0;
  if (s.rem > 0) {
    s.splits = cus / s.rem;  // (so rem * splits <= cus: the split round is one round)
    if (s.splits > MAX_STREAMK_SPLITS) s.splits = MAX_STREAMK_SPLITS;
    if (s.splits > k_tiles) s.splits = k_tiles;
    if (s.splits < 2) s.splits = 0;
  }
  return s;
}

size_t streamk_workspace_bytes(const StreamKPlan& plan) { return (size_t)plan.rem * plan.splits * SK_IMAGE_BYTES; }

int launch_streamk(const GemmParams& p, int64_t batch, int cus, void* workspace, size_t workspace_bytes, hipStream_t stream) {
  using C = CfgBig;
  if (p.K < C::BK || p.K % C::BK != 0 || p.M != p.N || p.M % C::TILE_M != 0 || p.M <= 0 || batch <= 0)
    return fail(MI_ERR_UNSUPPORTED_SHAPE, "internal: stream-K launch on %d x %d x %d", p.M, p.N, p.K);
  if (cus < 8 || cus % 8 != 0) return fail(MI_ERR_BAD_ARG, "internal: stream-K launch for %d CUs", cus);
  GemmParams q = p;
  q.tiles_m = q.tiles_n = p.M / C::TILE_M;
  const int64_t tiles = (int64_t)q.tiles_m * (q.tiles_m + 1) / 2 * batch;
  if (tiles / cus > 4096) return fail(MI_ERR_UNSUPPORTED_SHAPE, "internal: too many tiles for a stream-K launch");
  const StreamKPlan plan = streamk_plan(tiles, p.K / C::BK, cus);
  const size_t need = streamk_workspace_bytes(plan);
  if (need > 0 && (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u)))
    return fail(MI_ERR_WORKSPACE, "internal: stream-K workspace too small or misaligned");
  const bool split = plan.splits > 1;
  const int64_t whole = split ? (int64_t)plan.rounds * cus : tiles;  // (left-over tiles that are not split: one more round of whole tiles)
  if (whole > 0)
    if (int rc = launch_fast<C, false, false, MODE_SYRK, false>(p, batch, stream, whole)) return rc;
  int grid = g_last_launch.tiles;
  if (split) {
    q.lin_tiles = (int)whole;
    q.sk_rem = plan.rem;
    q.sk_splits = plan.splits;
    q.sk_tpx = (plan.rem + 7) / 8;
    q.sk_partials = static_cast<float*>(workspace);
    const int parts = 8 * q.sk_tpx * plan.splits;
    grid = (whole > 0 ? grid : 0) + parts;
    MI_LAUNCH_FAST(C, false, false, MODE_SYRK, false, false, SK_PARTS, false, dim3(parts), stream, q);
    MI_LAUNCH_FAST(CfgT128x2, false, false, MODE_SYRK, false, false, SK_FINISH, false, dim3(4 * plan.rem), stream, q);
  }
  g_last_launch = LastLaunch{grid, C::TILE_M, C::TILE_N, 2};
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
  return MI_OK;
}

}  // namespace mi
