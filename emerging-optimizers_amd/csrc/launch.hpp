// Host-side launchers of the tile engine.  The kernels are compiled in several translation units (one per kernel
// family, so that they build in parallel); each defines the launchers of its family by explicit instantiation of the
// templates in launch_impl.hpp, and the rest of the library only sees the declarations below.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm_fast.hpp"
#include "norm_common.hpp"

// Every launch of the fast kernel goes through MI_LAUNCH_FAST.  In the host-side bounds check build (MI_HOST_CHECK,
// `make host-check`) nothing is launched: the fast kernel's launches are walked on the host lane by lane
// (host_check.hpp); the other kernels' launches and the runtime calls around them are compiled out, and what is checked
// for them is the block of memory each pointer argument covers, which the launch site states with
//   MI_FOOTPRINT(what, base, bytes per element, batch, batch stride, rows, leading dimension, columns)
// (strides in elements; a null base states nothing).  In the ordinary build MI_FOOTPRINT and MI_OTHER_LAUNCH are empty.
#ifdef MI_HOST_CHECK
#include "host_check.hpp"
#undef hipLaunchKernelGGL
#define hipLaunchKernelGGL(...) ((void)0)
#define hipGetLastError() hipSuccess
#define hipFuncSetAttribute(...) hipSuccess
#define MI_LAUNCH_FAST(C, P_KS, Q_KS, MODE, OUT_F32, EDGE, SK, RMW, grid, stream, q) \
  ::mi::host_check::fast_launch<C, P_KS, Q_KS, MODE, OUT_F32, EDGE, SK, RMW>(grid, q)
#define MI_FOOTPRINT(...) ::mi::host_check::footprint(__VA_ARGS__)
#define MI_OTHER_LAUNCH() ::mi::host_check::other_launch()
#else
#define MI_FOOTPRINT(...) ((void)0)
#define MI_OTHER_LAUNCH() ((void)0)
#define MI_LAUNCH_FAST(C, P_KS, Q_KS, MODE, OUT_F32, EDGE, SK, RMW, grid, stream, q) \
  hipLaunchKernelGGL((gemm_fast_kernel<C, P_KS, Q_KS, MODE, OUT_F32, EDGE, SK, RMW>), grid, dim3(C::NT), 0, stream, q)
#endif

namespace mi {

// Records the text behind mi_last_error() for this host thread and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// What the last launch_one / launch_fast call on this thread launched: workgroups per batch entry and the tile shape.
struct LastLaunch {
  int tiles, tile_m, tile_n, fast;
};
extern thread_local LastLaunch g_last_launch;

// General kernel (gemm_engine.hpp): any multiple-of-8 shape, K tails, both operand layouts.
template <int BM, int BN, int BK, int WGM, int WGN, bool P_KS, bool Q_KS, int MODE, bool OUT_F32>
int launch_one(const GemmParams& p, int64_t batch, hipStream_t stream);

// Fast kernel (gemm_fast.hpp): K a multiple of the ring-slot depth; tiles that overhang the matrix only for the
// lower-triangle product of K-contiguous operands; anything else is refused with MI_ERR_UNSUPPORTED_SHAPE before
// a kernel is launched.
// A lower-triangle launch computes the tiles [0, tile_limit) of the batch, in the order of the kernel's numbering
// (tile_limit < 0: all of them).
template <class C, bool P_KS, bool Q_KS, int MODE, bool OUT_F32>
int launch_fast(const GemmParams& p, int64_t batch, hipStream_t stream, int64_t tile_limit = -1);

// CUs of the current device (cached).
int device_cus();

// 128-row matrices (inst_head_apply.hip): X' = beta X + alpha S X with S = p.P (128 x 128), X = p.Q (128 x p.N,
// row-major) and, when `gram_next` is given, the float32 partial Gram matrices of X' over slices of 512 columns
// ([batch][splits][128][128], lower-left three quadrants written).  One workgroup per (matrix, slice); scalars as in
// the GEMM mode of the tile engine, one partial sum of squares per workgroup at p.slots_out.
bool head_apply_supported(const GemmParams& p, int64_t batch, int splits);
int launch_head_apply(const GemmParams& p, int64_t batch, int splits, float* gram_next, bool out_f32, hipStream_t stream);

// 128-row matrices, first pass over the float32 input x ([batch][128][n], n a multiple of 512; with a momentum
// source, over the direction it defines, updating the buffer in place): the unnormalised bf16 copy to `xb`, one
// float64 partial sum of squares per (matrix, slice of 512 columns) to `partials`, and the float32 partial Gram
// matrices of the copy to `gram` (layout as above).  A second launch resolves the norm: norm[b], sumsq_out[b] (the
// squared norm of the normalised matrix) and xscale[b] = 1 / norm when the norm is in the range where the divide may
// be left to the consumers of X; outside it (xscale[b] = 1) that launch rewrites xb and `gram` from x / norm.
bool head_front_supported(const float* x, int64_t batch, int64_t n, const MomentumSrc& mom);
int launch_head_front(const float* x, int64_t batch, int64_t n, float eps, MomentumSrc mom, uint16_t* xb, double* partials,
                      float* gram, float* norm, float* sumsq_out, float* xscale, hipStream_t stream);

// Split-tail (stream-K) launch of the lower-triangle kernel (256 x 256 tiles, K-contiguous operands, bf16 output):
// with `cus` CUs (a multiple of 8), the whole rounds of `cus` tiles run one tile per workgroup, and the K range of each
// left-over tile is shared between `splits` workgroups (streamk_plan) that park their float32 accumulators in
// `workspace` (streamk_workspace_bytes), all in one launch; a second launch, one workgroup per left-over tile, adds
// the parked accumulators and writes the tile.
constexpr int MAX_STREAMK_SPLITS = 8;
struct StreamKPlan {
  int rounds, rem, splits;  // whole rounds of `cus` tiles, tiles left over, workgroups per left-over tile (0 or >= 2)
};
StreamKPlan streamk_plan(int64_t tiles, int k_tiles, int cus);
size_t streamk_workspace_bytes(const StreamKPlan& plan);
int launch_streamk(const GemmParams& p, int64_t batch, int cus, void* workspace, size_t workspace_bytes, hipStream_t stream);

}  // namespace mi
