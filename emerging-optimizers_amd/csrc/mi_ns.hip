// libmi_ns.so: C ABI over the gfx950 kernels (see include/mi_ns.h for the contract of each entry).
#include "../../include/mi_ns.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "launch.hpp"

namespace mi {

static thread_local std::string g_last_error;
thread_local LastLaunch g_last_launch = {0, 0, 0, 0};

int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

// ---------------------------------------------------------------------------------------------
// Process-wide options (mi_set_option / mi_get_option).  Each is one atomic integer; its initial value comes from an
// environment variable that is read once, when the first option is looked up.  Nothing on the call path reads the
// environment.
// ---------------------------------------------------------------------------------------------
enum Opt { OPT_STREAMK = 0, OPT_SYRK_TRANSPOSE, OPT_HEAD_APPLY, OPT_HEAD_FRONT, OPT_TALL_DIRECT, OPT_NS_PAIRS, OPT_COUNT };
struct OptDesc {
  const char* name;
  const char* env;
  int lo, hi, initial;
};
static constexpr OptDesc OPT_TABLE[OPT_COUNT] = {
    {"streamk", "MI_STREAMK", -1, 1, -1},                // -1 by the cost model, 0 never, 1 whenever the shape qualifies
    {"syrk_transpose", "MI_SYRK_TRANSPOSE", -1, 1, -1},  // -1 by the cost model, 0 never, 1 whenever the shape qualifies
    {"head_apply", "MI_HEAD_APPLY", 0, 1, 1},            // slab kernel for the B X product of 128-row matrices
    {"head_front", "MI_HEAD_FRONT", 0, 1, 1},            // input pass of 128-row matrices that leaves the Gram partials
    {"tall_direct", "MI_TALL_DIRECT", 0, 1, 1},          // last product of a tall input writes the result transposed
    {"ns_pairs", "MI_NS_PAIRS", -1, 2, -1},              // -1 by shape, 0 single steps, 1 never three at once, 2 pairs at every size
};
static std::atomic<int> g_opt[OPT_COUNT];
static std::once_flag g_opt_once;

static void opt_init() {
  std::call_once(g_opt_once, [] {
    for (int i = 0; i < OPT_COUNT; ++i) {
      int v = OPT_TABLE[i].initial;
      if (const char* e = getenv(OPT_TABLE[i].env)) {
        // numbers as they are; for MI_NS_PAIRS also the words "pairs" (1) and "force" (2)
        if (e[0] == 'p') v = 1;
        else if (e[0] == 'f') v = 2;
        else if ((e[0] >= '0' && e[0] <= '9') || e[0] == '-') v = atoi(e);
        if (v < OPT_TABLE[i].lo || v > OPT_TABLE[i].hi) v = OPT_TABLE[i].initial;
      }
      g_opt[i].store(v, std::memory_order_relaxed);
    }
  });
}
static int opt(Opt o) {
  opt_init();
  return g_opt[o].load(std::memory_order_relaxed);
}
static int opt_index(const char* name) {
  if (name)
    for (int i = 0; i < OPT_COUNT; ++i)
      if (strcmp(name, OPT_TABLE[i].name) == 0) return i;
  return -1;
}

// ---------------------------------------------------------------------------------------------
// Optional per-kernel timing of the fused driver: HIP event pairs recorded on the caller's stream.
// Off by default; mi_profile_begin() switches it on, mi_profile_end() waits for the events and reports.
// ---------------------------------------------------------------------------------------------
enum { PROF_NORMALIZE = 0, PROF_GRAM = 1, PROF_POLY = 2, PROF_APPLY = 3, PROF_KINDS = 4 };
struct ProfSpan {
  int kind;
  hipEvent_t start, stop;
};
static std::mutex g_prof_mutex;
static bool g_prof_on = false;
static std::vector<ProfSpan> g_prof_spans;

struct ProfScope {
  hipStream_t stream;
  hipEvent_t stop = nullptr;
  bool active = false;
  ProfScope(int kind, hipStream_t st) : stream(st) {
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    if (!g_prof_on) return;
    ProfSpan span{kind, nullptr, nullptr};
    if (hipEventCreate(&span.start) != hipSuccess || hipEventCreate(&span.stop) != hipSuccess) return;
    (void)hipEventRecord(span.start, stream);
    stop = span.stop;
    active = true;
    g_prof_spans.push_back(span);
  }
  ~ProfScope() {
    if (active) (void)hipEventRecord(stop, stream);
  }
};

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---------------------------------------------------------------------------------------------
// Tile-shape classes.  BIG is the MFMA-bound shape (one 4-wave workgroup per CU, 128 KB of LDS);
// MID/SMALL keep small and batched problems from launching mostly-empty tiles.
// ---------------------------------------------------------------------------------------------
enum TileClass { TILE_SMALL = 0, TILE_MID = 1, TILE_BIG = 2 };

static TileClass pick_class(int64_t extent) {
  if (extent >= 1024) return TILE_BIG;
  if (extent >= 256) return TILE_MID;
  return TILE_SMALL;
}

static int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Device-wide compute units (workgroups that run concurrently at one fast-kernel workgroup per CU).
int device_cus() {
  static int cached = 0;
  if (!cached) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      cached = n;
    else
      cached = 256;
  }
  return cached;
}

// Tile choice of the fast path by modelled time, fitted to measurements on this part.
//  * GEMM: 256 x 128 tiles cost about 1.27x per FLOP of 256 x 256 tiles and win when the latter leave CUs idle
//    (1024 x 4096: 64 tiles).
//  * Lower-triangle kernel (K-contiguous operands): a launch runs in rounds of g workgroups (one per CU; two for the
//    two-slot 128 x 128 tile), the last round possibly part-filled (share f of g).  In microseconds, with kt = 64-deep
//    K tiles:   L + full rounds x (F + s kt) + [last round] (F + min(s, s0 + s1 f) kt).
//    L is the launch, F prologue and write-out of a tile; the slope of a part-filled round is lower because the clock
//    follows the power drawn.  Least-squares fit over 437 shapes (n = 256 .. 8192, batch 1 .. 64, K = 256 .. 14336,
//    every tile forced in turn): relative error 3 - 8 % rms; the tile chosen is within 2 % of the best forced tile on
//    409 of them, 0.4 % slower on average, 18 % at worst (2 x 8192 x 256).
//                               L      F      s      s0     s1
//      128 x 128, one per CU   12.1    5.5   0.48   0.29   0.11     (n % 128 == 0)
//      128 x 128, two per CU    8.9    7.4   0.84   0.43   0.45     (n % 128 == 0; per pair of tiles)
//      192 x 192               14.6   10.8   0.79   0.50   0.26     (s was 0.81 in the fit; the loaders of edge tiles,
//                                                                 which most of the fitted shapes have, got cheaper since)
//      256 x 256               12.3   12.9   1.32   0.88   0.43     (n % 256 == 0)
//    Short K or few tiles favour the small tiles, long K with many tiles the 192 x 192 tile, and shapes whose
//    256 x 256 tiles fill whole rounds (8 x 1792: 224 tiles) or that 192 divides badly the 256 x 256 tile.
struct TileCost {
  double L, F, s, s0, s1;
  double operator()(int64_t count, int64_t g, double kt) const {
    const int64_t full = count / g, rem = count % g;
    return L + (double)full * (F + s * kt) + (rem ? F + std::min(s, s0 + s1 * (double)rem / (double)g) * kt : 0.0);
  }
};
static constexpr TileCost COST_128{12.1, 5.5, 0.48, 0.29, 0.11}, COST_128X2{8.9, 7.4, 0.84, 0.43, 0.45},
    COST_192{14.6, 10.8, 0.79, 0.50, 0.26}, COST_256{12.3, 12.9, 1.32, 0.88, 0.43};
enum SyrkTile { SYRK_TILE_NONE, SYRK_TILE_128, SYRK_TILE_128X2, SYRK_TILE_192, SYRK_TILE_256 };
// `k_strided`: the operand is stored transposed; its LDS layout exists for 128- and 256-row tiles only, and not for
// tiles that overhang the matrix, so there may be no fast tile at all.
static SyrkTile pick_syrk_tile(int64_t n, int64_t batch, int64_t k, bool k_strided, double* cost_us = nullptr) {
  const int64_t cus = device_cus();
  const double kt = (double)ceil_div(k, 64);
  auto tiles = [&](int64_t tile) {
    const int64_t t = ceil_div(n, tile);
    return t * (t + 1) / 2 * batch;
  };
  // (K-strided operands: full rounds at the slope of a full chip, the last partial round at the slope of its own fill)
  auto by_rounds = [&](int64_t count, double fixed, auto slope) {
    const int64_t full = count / cus, rem = count % cus;
    return (double)full * (fixed + slope(1.0) * kt) + (rem ? fixed + slope((double)rem / (double)cus) * kt : 0.0);
  };
  SyrkTile best = k_strided ? SYRK_TILE_NONE : SYRK_TILE_192;
  double best_cost = k_strided ? 1e30 : COST_192(tiles(192), cus, kt);
  auto offer = [&](SyrkTile t, double cost) {
    if (cost < best_cost) best = t, best_cost = cost;
  };
  if (k_strided) {
    // The transpose reads of a K-strided tile cost two LDS instructions per fragment: the K loop is 10 - 40 % slower
    // than on K-contiguous operands and hardly follows the fill (measured, n = 1024 .. 8192, K = 1024 .. 14336):
    //   256 x 256   s = 1.35 (f <= 0.55) .. 1.47      128 x 128, two per CU   0.90 per pair in a full round,
    //   128 x 128, one per CU   0.6 in a single round, 0.8 else             0.65 + 0.25 f in the last, partial one
    if (n % 256 == 0)
      offer(SYRK_TILE_256, by_rounds(tiles(256), 16.5, [](double f) { return f <= 0.55 ? 1.35 : 1.35 + (f - 0.55) * 0.27; }));
    if (n % 128 == 0) {
      const int64_t t128 = tiles(128), full = t128 / (2 * cus), rem = t128 % (2 * cus);
      offer(SYRK_TILE_128X2, (double)full * (9.2 + 0.90 * kt) +
                                 (rem ? 9.2 + (0.65 + 0.25 * (double)rem / (double)(2 * cus)) * kt : 0.0));
      offer(SYRK_TILE_128, t128 <= cus ? 9.0 + 0.6 * kt : (double)ceil_div(t128, cus) * (9.0 + 0.8 * kt));
    }
    if (cost_us) *cost_us = best_cost;
    return best;
  }
  if (n % 256 == 0) offer(SYRK_TILE_256, COST_256(tiles(256), cus, kt));
  if (n % 128 == 0) {
    offer(SYRK_TILE_128X2, COST_128X2(tiles(128), 2 * cus, kt));
    offer(SYRK_TILE_128, COST_128(tiles(128), cus, kt));
  }
  if (cost_us) *cost_us = best_cost;
  return best;
}

// Split-tail (stream-K) launch of the lower-triangle kernel (256 x 256 tiles; whole rounds of tiles, then the
// left-over tiles with their K range split between workgroups): true when the shape qualifies and the model
// expects a gain over the best ordinary launch; `plan` is filled either way.  Modelled time: the whole rounds and the
// split round as launches of 256 x 256 tiles, and the finishing launch (8 us, and 3 us per accumulator image it
// adds; 20 us measured for 64 tiles of 4 images).
static int streamk_cus() { return device_cus() / 8 * 8; }
static bool streamk_wanted(int64_t n, int64_t batch, int64_t k, bool k_strided, StreamKPlan* plan) {
  *plan = StreamKPlan{0, 0, 0};
  const int cus = streamk_cus();
  if (k_strided || n < 1024 || n % 256 != 0 || k % 64 != 0 || k < 64 || cus < 8) return false;
  const int mode = opt(OPT_STREAMK);  // 0: never, 1: whenever the shape qualifies (tests), else by the model
  if (mode == 0) return false;
  const int64_t t = n / 256, tiles = t * (t + 1) / 2 * batch, kt = k / 64;
  if (tiles / cus > 4096) return false;
  *plan = streamk_plan(tiles, (int)kt, cus);
  if (mode == 1) return true;
  if (plan->splits < 2) return false;
  double best = 0.0;
  pick_syrk_tile(n, batch, k, false, &best);
  const double sk = (plan->rounds ? COST_256((int64_t)plan->rounds * cus, cus, (double)kt) : 0.0) +
                    COST_256((int64_t)plan->rem * plan->splits, cus, (double)ceil_div(kt, plan->splits)) + 8.0 + 3.0 * plan->splits;
  return sk < 0.97 * best;
}
// 256 x 128 instead of 256 x 256 GEMM tiles for the whole product?
static bool gemm_prefers_half_tiles(int64_t m, int64_t n, int64_t batch) {
  const int64_t cus = device_cus(), tiles = (m / 256) * (n / 256) * batch;
  return (double)ceil_div(2 * tiles, cus) * 0.5 * 1.27 < (double)ceil_div(tiles, cus);
}

// Whether the float32 GEMM+AXPY of an (m x m) by (m x n) product runs on kernels that can write their result
// transposed (the staged epilogue of the fast kernel; mirrors the choices of launch_class below).
static bool gemm_transposed_out_ok(int64_t m, int64_t n) {
  if (m % 64 != 0 || m < 64) return false;
  if (m >= (1 << 22) || n >= (1 << 22)) return false;  // (launch_class: such leading dimensions stay on the general kernel)
  if (m >= 1024 && n >= 1024 && m % 256 == 0 && n % 256 == 0) return true;
  return m % 128 == 0 && m < 1024 && n % 256 == 0 && n >= 256;
}

template <bool P_KS, bool Q_KS, int MODE, bool OUT_F32>
static int launch_class(TileClass tc, const GemmParams& p, int64_t batch, hipStream_t stream) {
  const bool k_ok = p.K % 64 == 0 && p.K >= 64;
  // Lower-triangle products of 256 rows and more whose rows are whole 128-row tiles also take the direct-to-LDS
  // kernels (general kernel 1.25 - 2.45x slower over 129 shapes, n = 256 .. 768, batch 1 .. 64); other small
  // matrices stay on the general kernel.
  // (leading dimensions beyond 4M elements -- a 4096-row bf16 operand of more than 32 GB -- stay on the general kernel:
  // the fast loaders address the rows of a tile with 32-bit byte offsets)
  const bool ld_ok = p.ldp < (1 << 22) && p.ldq < (1 << 22);
  const bool big = ld_ok && ((p.M >= 1024 && p.N >= 1024) || (MODE == MODE_SYRK && p.M >= 256 && p.M % 128 == 0));
  if (k_ok && big) {
    if constexpr (MODE == MODE_SYRK) {
      static_assert(P_KS == Q_KS, "the lower-triangle product reads one operand in one layout");
      switch (pick_syrk_tile(p.M, batch, p.K, P_KS)) {
        case SYRK_TILE_128:
          return launch_fast<CfgT128, P_KS, Q_KS, MODE, OUT_F32>(p, batch, stream);
        case SYRK_TILE_128X2:
          return launch_fast<CfgT128x2, P_KS, Q_KS, MODE, OUT_F32>(p, batch, stream);
        case SYRK_TILE_256:
          return launch_fast<CfgBig, P_KS, Q_KS, MODE, OUT_F32>(p, batch, stream);
        case SYRK_TILE_192:
          if constexpr (!P_KS) return launch_fast<CfgSyrk192, false, false, MODE, OUT_F32>(p, batch, stream);
          break;
        default:
          break;  // no fast tile for this shape: the general kernel below
      }
    }
    if constexpr (MODE == MODE_GEMM && !P_KS && Q_KS) {
      if (big && p.M % 256 == 0 && p.N % 256 == 0 && gemm_prefers_half_tiles(p.M, p.N, batch))
        return launch_fast<CfgHalfN, false, true, MODE, OUT_F32>(p, batch, stream);
    }
    if constexpr (MODE == MODE_GEMM) {
      if (big && p.M % 256 == 0 && p.N % 256 == 0) return launch_fast<CfgBig, P_KS, Q_KS, MODE, OUT_F32>(p, batch, stream);
    }
  }
  if constexpr (MODE == MODE_GEMM && !P_KS && Q_KS) {
    // short, wide products (per-head shapes): 128 x 256 tiles keep the direct-to-LDS loads and the coalesced epilogue
    if (k_ok && p.M % 128 == 0 && p.M < 1024 && p.N % 256 == 0 && p.N >= 256)
      return launch_fast<CfgM128, false, true, MODE, OUT_F32>(p, batch, stream);
  }
  switch (tc) {
    case TILE_BIG:
      return launch_one<256, 256, 64, 2, 2, P_KS, Q_KS, MODE, OUT_F32>(p, batch, stream);
    case TILE_MID:
      return launch_one<128, 128, 64, 2, 2, P_KS, Q_KS, MODE, OUT_F32>(p, batch, stream);
    default:
      return launch_one<64, 64, 64, 2, 2, P_KS, Q_KS, MODE, OUT_F32>(p, batch, stream);
  }
}

// Diagonal-shift wiring of one launch inside the fused driver (see GemmParams).
struct ShiftArgs {
  int mode;
  float cb, cc;
  const float* slots_in;
  int nslots_in;
  float* shift_io;
  float* slots_out;
  const float* group_abc = nullptr;  // SHIFT_GROUP_*: (a, b, c) of the steps of the group, 3 floats each
  int group_size = 0, stage = 0;
  const float* xscale = nullptr;  // first group of steps on an unnormalised X
  int slot_capacity = 0;          // floats reserved per batch entry behind slots_out
  void apply(GemmParams& p) const {
    p.shift_mode = mode;
    p.xscale = xscale;
    p.ca = 0.0f;
    p.cb = cb;
    p.cc = cc;
    for (int j = 0; j < 3; ++j)
      for (int e = 0; e < 3; ++e) p.co[j][e] = (group_abc && j < group_size) ? group_abc[3 * j + e] : 0.0f;
    p.stage = stage;
    p.slots_in = slots_in;
    p.nslots_in = nslots_in;
    p.shift_io = shift_io;
    p.slots_out = slots_out;
    p.slot_stride = 0;  // filled in by the launcher
    p.slot_base = 0;
    p.slot_capacity = slot_capacity;
  }
};

// D = alpha * A A^T + beta * C, bf16 out.
// Inside the fused driver the same lower-triangle kernel also forms products of two commuting symmetric matrices:
// dst[b][r][c] = src[b][c][r] for bf16 matrices: src has `cols_out` rows of `rows_out` elements.  64 x 64 tiles through LDS,
// 16-byte global accesses on both sides (all extents are multiples of 8).
__global__ void __launch_bounds__(256) transpose_bf16_kernel(const uint16_t* __restrict__ src, int64_t src_bs, int64_t src_ld,
                                                             uint16_t* __restrict__ dst, int64_t dst_bs, int64_t dst_ld,
                                                             int rows_out, int cols_out) {
  __shared__ uint16_t tile[64][64 + 2];  // [row of dst][column of dst]; 33 words per row: conflict-free column writes
  const int r0 = blockIdx.x * 64, c0 = blockIdx.y * 64, tid = threadIdx.x;
  const uint16_t* s = src + blockIdx.z * src_bs;
  uint16_t* d = dst + blockIdx.z * dst_bs;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int ch = tid + 256 * i, c = ch / 8, r = (ch % 8) * 8;  // source row c0 + c, elements r0 + r .. + 7
    if (c0 + c < cols_out && r0 + r < rows_out) {
      const uint4 v = *reinterpret_cast<const uint4*>(s + (int64_t)(c0 + c) * src_ld + r0 + r);
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        tile[r + 2 * e][c] = (uint16_t)(w[e] & 0xffffu);
        tile[r + 2 * e + 1][c] = (uint16_t)(w[e] >> 16);
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int ch = tid + 256 * i, r = ch / 8, c = (ch % 8) * 8;
    if (r0 + r < rows_out && c0 + c < cols_out) {
      uint32_t w[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) w[e] = (uint32_t)tile[r][c + 2 * e] | ((uint32_t)tile[r][c + 2 * e + 1] << 16);
      *reinterpret_cast<uint4*>(d + (int64_t)(r0 + r) * dst_ld + c0 + c) = make_uint4(w[0], w[1], w[2], w[3]);
    }
  }
}

// A K-strided operand of a lower-triangle product (stored as K rows of N): copy it transposed into scratch memory
// first?  The K loop of the K-strided kernels is slower and they have no 192 x 192 tile; the copy runs at about
// 4 TB/s (read + write).  Bytes of scratch the copy needs, or 0 when the model expects no gain.
static size_t transposed_copy_bytes(int64_t n, int64_t batch, int64_t k) {
  if (n < 1024 || k % 64 != 0) return 0;  // (below, both layouts go to the general kernel)
  const int mode = opt(OPT_SYRK_TRANSPOSE);  // 0: never, 1: always (tests), else by the model
  if (mode == 0) return 0;
  const size_t bytes = ((size_t)batch * n * k * 2 + 255) / 256 * 256;
  if (mode == 1) return bytes;
  if (n < 2048) return 0;  // (launches of a few dozen small tiles: the model is too coarse there, measured no gain)
  double strided = 0.0, contiguous = 0.0;
  if (pick_syrk_tile(n, batch, k, true, &strided) == SYRK_TILE_NONE) return bytes;
  pick_syrk_tile(n, batch, k, false, &contiguous);
  const double copy = 6.0 + 2.0 * (double)bytes / 4.0e6;
  return contiguous + copy < 0.95 * strided ? bytes : 0;
}

// Argument checks of the lower-triangle product, shared by every entry that leads to it: nothing is launched for a
// call that fails one of them.
static int syrk_validate(const void* A, int64_t batch, int64_t n, int64_t k, int64_t a_bs, int64_t a_ld, int a_trans,
                         const void* C, int64_t c_bs, int64_t c_ld, float beta, const void* D, int64_t d_bs, int64_t d_ld) {
  if (!A || !D) return fail(MI_ERR_BAD_ARG, "mi_syrk_bf16: A and D must not be null");
  if (batch < 0 || n < 0 || k < 0) return fail(MI_ERR_BAD_ARG, "mi_syrk_bf16: negative extent");
  if (beta != 0.0f && !C) return fail(MI_ERR_BAD_ARG, "mi_syrk_bf16: C is null but beta != 0");
  if (n % 8 || k % 8) return fail(MI_ERR_UNSUPPORTED_SHAPE, "N and K must be multiples of 8, got N=%lld, K=%lld", (long long)n, (long long)k);
  if (a_ld % 8 || d_ld % 8 || a_bs % 8 || d_bs % 8 || (C && (c_ld % 8 || c_bs % 8)))
    return fail(MI_ERR_UNSUPPORTED_SHAPE, "mi_syrk_bf16: leading dimensions and batch strides must be multiples of 8");
  if (!aligned16(A) || !aligned16(D) || (C && !aligned16(C)))
    return fail(MI_ERR_UNSUPPORTED_SHAPE, "mi_syrk_bf16: pointers must be 16-byte aligned");
  if (a_ld < (a_trans ? n : k) || d_ld < n || (C && c_ld < n)) return fail(MI_ERR_BAD_ARG, "mi_syrk_bf16: leading dimension too small");
  if (n > (1 << 30) || k > (1 << 30)) return fail(MI_ERR_UNSUPPORTED_SHAPE, "mi_syrk_bf16: extent too large");
  return MI_OK;
}

// `other` != null computes alpha * A other^T (symmetric in exact arithmetic; the lower triangle is computed and
// mirrored), and `C2` is a second addend laid out like C whose coefficient a SHIFT_GROUP_* mode supplies.
static int syrk_impl(const void* A, int64_t batch, int64_t n, int64_t k, int64_t a_bs, int64_t a_ld, int a_trans,
                     const void* C, int64_t c_bs, int64_t c_ld, float alpha, float beta, void* D, int64_t d_bs,
                     int64_t d_ld, int skip_upper, hipStream_t stream, const ShiftArgs* sh = nullptr,
                     const void* other = nullptr, const void* C2 = nullptr, void* workspace = nullptr,
                     size_t workspace_bytes = 0) {
  if (int rc = syrk_validate(A, batch, n, k, a_bs, a_ld, a_trans, C, c_bs, c_ld, beta, D, d_bs, d_ld)) return rc;
  if (batch == 0 || n == 0) return MI_OK;

  GemmParams p{};
  p.P = static_cast<const uint16_t*>(A);
  p.Q = other ? static_cast<const uint16_t*>(other) : p.P;
  p.Cin2 = static_cast<const uint16_t*>(C2);
  p.beta2 = C2 ? 1.0f : 0.0f;  // replaced by the shift mode
  p.ldp = p.ldq = a_ld;
  p.p_bs = p.q_bs = a_bs;
  p.Cin = (beta != 0.0f) ? static_cast<const uint16_t*>(C) : nullptr;
  p.ldc = c_ld;
  p.c_bs = c_bs;
  p.Out = D;
  p.ldo = d_ld;
  p.o_bs = d_bs;
  p.M = p.N = (int)n;
  p.K = (int)k;
  p.alpha = alpha;
  p.beta = beta;
  p.out_scale = 1.0f;
  p.skip_upper = skip_upper ? 1 : 0;
  if (sh) sh->apply(p);
  // With a workspace, shapes whose tiles fill the chip's rounds badly go out as a split-tail launch.
  if (!skip_upper && sh == nullptr && C2 == nullptr) {
    StreamKPlan plan;
    if (streamk_wanted(n, batch, k, a_trans != 0, &plan)) {
      const size_t need = streamk_workspace_bytes(plan);
      if (need == 0 || (workspace != nullptr && workspace_bytes >= need && !(reinterpret_cast<uintptr_t>(workspace) & 255u)))
        return launch_streamk(p, batch, streamk_cus(), workspace, workspace_bytes, stream);
    }
  }
  TileClass tc = pick_class(n);
  return a_trans ? launch_class<true, true, MODE_SYRK, false>(tc, p, batch, stream)
                 : launch_class<false, false, MODE_SYRK, false>(tc, p, batch, stream);
}

// Xout = beta * X + alpha * (Bm X)
static int gemm_axpy_impl(const void* Bm, int64_t b_bs, int64_t b_ld, const void* X, int64_t x_bs,
                          int64_t x_ld, int x_trans, void* Xout, int64_t o_bs, int64_t o_ld, int64_t batch,
                          int64_t m, int64_t n, float alpha, float beta, int out_fp32, float out_scale,
                          hipStream_t stream, const ShiftArgs* sh = nullptr, float out_accum = 0.0f, int head_splits = 0,
                          float* head_gram_next = nullptr, bool* head_used = nullptr, int out_transposed = 0) {
  if (!Bm || !X || !Xout) return fail(MI_ERR_BAD_ARG, "mi_gemm_axpy_bf16: null pointer");
  if (batch < 0 || m < 0 || n < 0) return fail(MI_ERR_BAD_ARG, "mi_gemm_axpy_bf16: negative extent");
  if (m % 8 || n % 8) return fail(MI_ERR_UNSUPPORTED_SHAPE, "M and N must be multiples of 8, got M=%lld, N=%lld", (long long)m, (long long)n);
  if (b_ld % 8 || x_ld % 8 || b_bs % 8 || x_bs % 8 || o_ld % 4 || o_bs % 4)
    return fail(MI_ERR_UNSUPPORTED_SHAPE, "mi_gemm_axpy_bf16: leading dimensions and batch strides must be multiples of 8");
  if (!aligned16(Bm) || !aligned16(X) || !aligned16(Xout))
    return fail(MI_ERR_UNSUPPORTED_SHAPE, "mi_gemm_axpy_bf16: pointers must be 16-byte aligned");
  const int64_t x_inner = x_trans ? m : n;
  if (out_transposed && (x_trans || !out_fp32)) return fail(MI_ERR_BAD_ARG, "internal: transposed output of this product");
  if (b_ld < m || x_ld < x_inner || o_ld < (out_transposed ? m : x_inner))
    return fail(MI_ERR_BAD_ARG, "mi_gemm_axpy_bf16: leading dimension too small");
  if (m > (1 << 30) || n > (1 << 30)) return fail(MI_ERR_UNSUPPORTED_SHAPE, "mi_gemm_axpy_bf16: extent too large");
  if (batch == 0 || m == 0 || n == 0) return MI_OK;

  GemmParams p{};
  p.Cin = (beta != 0.0f) ? static_cast<const uint16_t*>(X) : nullptr;
  p.ldc = x_ld;
  p.c_bs = x_bs;
  p.Out = Xout;
  p.ldo = o_ld;
  p.o_bs = o_bs;
  p.K = (int)m;
  p.alpha = alpha;
  p.beta = beta;
  p.out_scale = out_scale;
  p.out_accum = out_fp32 ? out_accum : 0.0f;
  p.out_transposed = out_transposed;
  if (sh) sh->apply(p);
  TileClass tc = pick_class(m);
  if (!x_trans) {
    // OUT (m x n): P = Bm rows (K-contiguous), Q[j][k] = X[k][j] (K-strided).
    p.P = static_cast<const uint16_t*>(Bm);
    p.ldp = b_ld;
    p.p_bs = b_bs;
    p.Q = static_cast<const uint16_t*>(X);
    p.ldq = x_ld;
    p.q_bs = x_bs;
    p.M = (int)m;
    p.N = (int)n;
    // 128-row matrices inside the driver: one workgroup per 512-column slice does product, addend and the next
    // group's partial Gram matrices on slabs it keeps in LDS
    // (option "head_apply" = 0: the general GEMM+AXPY kernels also for 128-row matrices -- A/B runs, tests)
    if (head_splits > 0 && opt(OPT_HEAD_APPLY) != 0 && head_apply_supported(p, batch, head_splits)) {
      if (head_used) *head_used = true;
      return launch_head_apply(p, batch, head_splits, out_fp32 ? nullptr : head_gram_next, out_fp32 != 0, stream);
    }
    // Tile-count quantisation: T full 256 x 256 tiles over C compute units leave a last round that is at most half
    // full when 0 < T mod C <= C/2.  If that remainder is a whole number of tile columns or of tile rows (of every
    // matrix of the batch), those run as 256 x 128 tiles in a second launch: twice as many workgroups, one short round
    // (4096 x 14336: 768 + 256 workgroups instead of 896; 8 x 1792 x 4096: the last tile row of every matrix).
    if (m % 256 == 0 && n % 256 == 0 && m >= 1024 && n >= 1024 && !gemm_prefers_half_tiles(m, n, batch)) {
      const int64_t tm = m / 256, tn = n / 256, cus = device_cus();
      const int64_t rem = (tm * tn * batch) % cus;
      int64_t tail_cols = 0, tail_rows = 0;
      if (rem > 0 && rem * 2 <= cus) {
        if (rem % (tm * batch) == 0 && rem / (tm * batch) < tn) tail_cols = rem / (tm * batch) * 256;
        else if (rem % (tn * batch) == 0 && rem / (tn * batch) < tm) tail_rows = rem / (tn * batch) * 256;
      }
      if (tail_cols > 0 || tail_rows > 0) {
        const int64_t main_cols = n - tail_cols, main_rows = m - tail_rows;
        // per matrix: workgroups of the main launch, then those of the tail launch
        const int tiles_main = (int)((main_rows / 256) * (main_cols / 256));
        const int tiles_tail = (int)(tail_cols ? tm * (tail_cols / 128) : (tail_rows / 256) * (n / 128));
        GemmParams pm = p, pt = p;
        pm.slot_stride = pt.slot_stride = tiles_main + tiles_tail;
        pm.slot_base = 0;
        pt.slot_base = tiles_main;
        int64_t out_off = 0;
        if (tail_cols) {
          pm.N = (int)main_cols;
          pt.N = (int)tail_cols;
          pt.Q = p.Q + main_cols;  // K-strided operand: column offset
          if (pt.Cin) pt.Cin = p.Cin + main_cols;
          out_off = out_transposed ? main_cols * p.ldo : main_cols;
        } else {
          pm.M = (int)main_rows;
          pt.M = (int)tail_rows;
          pt.P = p.P + main_rows * p.ldp;
          if (pt.Cin) pt.Cin = p.Cin + main_rows * p.ldc;
          out_off = out_transposed ? main_rows : main_rows * p.ldo;
        }
        pt.Out = out_fp32 ? static_cast<void*>(static_cast<float*>(p.Out) + out_off)
                          : static_cast<void*>(static_cast<uint16_t*>(p.Out) + out_off);
        int rc = out_fp32 ? launch_fast<CfgBig, false, true, MODE_GEMM, true>(pm, batch, stream)
                          : launch_fast<CfgBig, false, true, MODE_GEMM, false>(pm, batch, stream);
        if (rc != MI_OK) return rc;
        rc = out_fp32 ? launch_fast<CfgHalfN, false, true, MODE_GEMM, true>(pt, batch, stream)
                      : launch_fast<CfgHalfN, false, true, MODE_GEMM, false>(pt, batch, stream);
        g_last_launch.tiles = tiles_main + tiles_tail;
        return rc;
      }
    }
    return out_fp32 ? launch_class<false, true, MODE_GEMM, true>(tc, p, batch, stream)
                    : launch_class<false, true, MODE_GEMM, false>(tc, p, batch, stream);
  }
  // Memory holds X^T (n x m): OUT^T[j][i] = sum_k X^T[j][k] * Bm[i][k], both operands K-contiguous.
  p.P = static_cast<const uint16_t*>(X);
  p.ldp = x_ld;
  p.p_bs = x_bs;
  p.Q = static_cast<const uint16_t*>(Bm);
  p.ldq = b_ld;
  p.q_bs = b_bs;
  p.M = (int)n;
  p.N = (int)m;
  return out_fp32 ? launch_class<false, false, MODE_GEMM, true>(tc, p, batch, stream)
                  : launch_class<false, false, MODE_GEMM, false>(tc, p, batch, stream);
}

// ---------------------------------------------------------------------------------------------
// Frobenius normalisation: a sum-of-squares pass that leaves one partial per workgroup, and a
// scale/cast pass whose workgroups each re-add those partials in a fixed order (deterministic,
// no atomics, no extra launch for the final reduction).
// ---------------------------------------------------------------------------------------------
static constexpr int NORM_THREADS = 256;
static constexpr int NORM_MAX_BLOCKS = 1024;  // partials per matrix

static int norm_blocks(int64_t numel) {
  int64_t vec = numel / 4;  // float4 units
  int64_t want = (vec + (int64_t)NORM_THREADS * 8 - 1) / ((int64_t)NORM_THREADS * 8);
  if (want < 1) want = 1;
  if (want > NORM_MAX_BLOCKS) want = NORM_MAX_BLOCKS;
  return (int)want;
}

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;
}

template <typename T>
__device__ __forceinline__ T block_sum(T v, T* scratch) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  T total = 0;
  if (threadIdx.x == 0) {
    for (int w = 0; w < NORM_THREADS / 64; ++w) total += scratch[w];
    scratch[0] = total;
  }
  __syncthreads();
  total = scratch[0];
  __syncthreads();
  return total;
}

__device__ __forceinline__ float4 stream_load(const float4* p) {
  const f32x4_t t = stream_load4(reinterpret_cast<const float*>(p));
  return make_float4(t[0], t[1], t[2], t[3]);
}

// `raw_out` != null: the values that are summed are also written out as bf16, unnormalised (bf16 has the exponent
// range of float32, so this loses nothing that the later divide would keep).
template <bool F64>
__global__ void __launch_bounds__(NORM_THREADS) sumsq_kernel(const float* __restrict__ x, int64_t numel,
                                                             double* __restrict__ partials, MomentumSrc mom,
                                                             uint16_t* __restrict__ raw_out) {
  const int64_t b = blockIdx.y;
  uint2* __restrict__ rv = raw_out ? reinterpret_cast<uint2*>(raw_out + b * numel) : nullptr;
  const float4* __restrict__ xv = reinterpret_cast<const float4*>(x + b * numel);
  float4* __restrict__ bv = mom.buf ? reinterpret_cast<float4*>(mom.buf + b * numel) : nullptr;
  const int64_t nvec = numel / 4;
  // with a momentum source: update the buffer in place and return the direction whose norm is wanted
  auto fetch = [&](int64_t i) {
    float4 v = stream_load(xv + i);
    if (bv) {
      float4 m = bv[i];
      m.x = torch_lerp(m.x, v.x, 1.0f - mom.beta);
      m.y = torch_lerp(m.y, v.y, 1.0f - mom.beta);
      m.z = torch_lerp(m.z, v.z, 1.0f - mom.beta);
      m.w = torch_lerp(m.w, v.w, 1.0f - mom.beta);
      bv[i] = m;
      v.x = momentum_direction(v.x, m.x, mom.beta, mom.nesterov);
      v.y = momentum_direction(v.y, m.y, mom.beta, mom.nesterov);
      v.z = momentum_direction(v.z, m.z, mom.beta, mom.nesterov);
      v.w = momentum_direction(v.w, m.w, mom.beta, mom.nesterov);
    }
    if (rv) {
      const f32x4_t f = {v.x, v.y, v.z, v.w};
      rv[i] = __builtin_bit_cast(uint2, __builtin_convertvector(f, bf16x4_t));
    }
    return v;
  };
  const int64_t stride = (int64_t)gridDim.x * NORM_THREADS;
  __shared__ double scratch_d[NORM_THREADS / 64];
  double total;
  if (F64) {
    double s0 = 0, s1 = 0, s2 = 0, s3 = 0;
    for (int64_t i = (int64_t)blockIdx.x * NORM_THREADS + threadIdx.x; i < nvec; i += stride) {
      float4 v = fetch(i);
      s0 += (double)v.x * (double)v.x;
      s1 += (double)v.y * (double)v.y;
      s2 += (double)v.z * (double)v.z;
      s3 += (double)v.w * (double)v.w;
    }
    total = block_sum<double>((s0 + s1) + (s2 + s3), scratch_d);
  } else {
    float s0 = 0, s1 = 0, s2 = 0, s3 = 0;
    int64_t i = (int64_t)blockIdx.x * NORM_THREADS + threadIdx.x;
    // four independent 16-byte loads in flight per lane: a single one leaves HBM latency exposed (more change nothing)
    constexpr int UNROLL = 4;
    for (; i + (UNROLL - 1) * stride < nvec; i += UNROLL * stride) {
      float4 v[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) v[u] = fetch(i + u * stride);
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        s0 = __builtin_fmaf(v[u].x, v[u].x, s0); s1 = __builtin_fmaf(v[u].y, v[u].y, s1);
        s2 = __builtin_fmaf(v[u].z, v[u].z, s2); s3 = __builtin_fmaf(v[u].w, v[u].w, s3);
      }
    }
    for (; i < nvec; i += stride) {
      float4 v = fetch(i);
      s0 = __builtin_fmaf(v.x, v.x, s0);
      s1 = __builtin_fmaf(v.y, v.y, s1);
      s2 = __builtin_fmaf(v.z, v.z, s2);
      s3 = __builtin_fmaf(v.w, v.w, s3);
    }
    // squares are formed in float32 (tiny inputs underflow exactly like a float32 reduction);
    // the cross-thread tree is carried in float64 so the result does not depend on its shape.
    total = block_sum<double>((double)((s0 + s1) + (s2 + s3)), scratch_d);
  }
  if (threadIdx.x == 0) partials[b * gridDim.x + blockIdx.x] = total;
}

template <bool F64, bool OUT_BF16>
__global__ void __launch_bounds__(NORM_THREADS) scale_cast_kernel(const float* __restrict__ x, int64_t numel,
                                                                  const double* __restrict__ partials, int nparts,
                                                                  float eps, float post_scale, void* __restrict__ out,
                                                                  float* __restrict__ dev_norm,
                                                                  float* __restrict__ sumsq_out, MomentumSrc mom,
                                                                  float* __restrict__ xscale) {
  const int64_t b = blockIdx.y;
  __shared__ double scratch_d[NORM_THREADS / 64];
  double s = 0;
  for (int i = threadIdx.x; i < nparts; i += NORM_THREADS) s += partials[b * nparts + i];
  s = block_sum<double>(s, scratch_d);
  float divisor;
  if (F64) {
    divisor = (float)sqrt(s);
  } else {
    divisor = fmaxf(sqrtf((float)s), eps);
  }
  if (dev_norm && blockIdx.x == 0 && threadIdx.x == 0) dev_norm[b] = divisor;
  // `xscale` != null: `out` already holds the unnormalised bf16 values (sumsq_kernel wrote them).  For a norm in
  // the range where squares of the entries neither overflow nor vanish in float32 the divide is left to the
  // kernels that consume X (they multiply by xscale) and this pass ends here; otherwise it normalises as usual.
  bool deferred = false;
  if (xscale) {
    deferred = divisor >= NORM_DEFER_MIN && divisor <= NORM_DEFER_MAX;  // false for NaN
    if (blockIdx.x == 0 && threadIdx.x == 0) xscale[b] = deferred ? 1.0f / divisor : 1.0f;
  }
  if (sumsq_out && blockIdx.x == 0 && threadIdx.x == 0) {
    // squared Frobenius norm of the normalised matrix: 1 unless the divisor was clamped
    const float ratio = sqrtf((float)s) / divisor;
    sumsq_out[b] = (divisor > 0.0f && ratio == ratio) ? ratio * ratio : 0.0f;
  }
  if (deferred) return;

  const int64_t nvec8 = numel / 8;
  const float4* __restrict__ xv = reinterpret_cast<const float4*>(x + b * numel);
  const float4* __restrict__ bv = mom.buf ? reinterpret_cast<const float4*>(mom.buf + b * numel) : nullptr;
  auto fetch = [&](int64_t i) {  // the direction again, from the buffer the first pass already updated
    float4 v = xv[i];
    if (bv) {
      const float4 m = bv[i];
      v.x = momentum_direction(v.x, m.x, mom.beta, mom.nesterov);
      v.y = momentum_direction(v.y, m.y, mom.beta, mom.nesterov);
      v.z = momentum_direction(v.z, m.z, mom.beta, mom.nesterov);
      v.w = momentum_direction(v.w, m.w, mom.beta, mom.nesterov);
    }
    return v;
  };
  const int64_t stride = (int64_t)gridDim.x * NORM_THREADS;
  for (int64_t i = (int64_t)blockIdx.x * NORM_THREADS + threadIdx.x; i < nvec8; i += stride) {
    float4 a = fetch(2 * i), c = fetch(2 * i + 1);
    f32x4_t lo = {a.x / divisor, a.y / divisor, a.z / divisor, a.w / divisor};
    f32x4_t hi = {c.x / divisor, c.y / divisor, c.z / divisor, c.w / divisor};
    if (OUT_BF16) {
      bf16x4_t hl = __builtin_convertvector(lo, bf16x4_t);
      bf16x4_t hh = __builtin_convertvector(hi, bf16x4_t);
      uint2 ul = __builtin_bit_cast(uint2, hl), uh = __builtin_bit_cast(uint2, hh);
      reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(out) + b * numel)[i] = make_uint4(ul.x, ul.y, uh.x, uh.y);
    } else {
      f32x4_t* o = reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(out) + b * numel);
      o[2 * i] = lo * post_scale;
      o[2 * i + 1] = hi * post_scale;
    }
  }
}

// Tall inputs (rows > cols): the bf16 cast also transposes, so that the iteration can run on the (cols x rows)
// orientation with K-contiguous operands (the fastest kernels), and the float32 result is transposed back once at
// the end.  64 x 64 tiles through LDS, 16-byte global accesses on both sides; every workgroup walks over tiles
// blockIdx.x, blockIdx.x + gridDim.x, ...
struct TileWalk {
  int64_t rows, cols;
  int tiles_c;
  int64_t ntiles;
  __device__ TileWalk(int64_t r, int64_t c) : rows(r), cols(c), tiles_c((int)((c + 63) / 64)), ntiles(((r + 63) / 64) * ((c + 63) / 64)) {}
};
// One 64 x 64 tile of `tile` (float32, [row][col]) -> bf16 at out[(c0 + c) * rows + r0 + r], values divided by `div`.
__device__ __forceinline__ void store_tile_transposed(const float (&tile)[64][65], uint16_t* __restrict__ ob, int64_t rows,
                                                      int64_t cols, int64_t r0, int64_t c0, float div) {
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int c = pass * 32 + (threadIdx.x >> 3), r = (threadIdx.x & 7) * 8;
    if (c0 + c < cols && r0 + r < rows) {
      f32x4_t lo = {tile[r][c] / div, tile[r + 1][c] / div, tile[r + 2][c] / div, tile[r + 3][c] / div};
      f32x4_t hi = {tile[r + 4][c] / div, tile[r + 5][c] / div, tile[r + 6][c] / div, tile[r + 7][c] / div};
      const uint2 a = __builtin_bit_cast(uint2, __builtin_convertvector(lo, bf16x4_t));
      const uint2 d = __builtin_bit_cast(uint2, __builtin_convertvector(hi, bf16x4_t));
      *reinterpret_cast<uint4*>(ob + (c0 + c) * rows + r0 + r) = make_uint4(a.x, a.y, d.x, d.y);
    }
  }
}

// First pass of a tall input when the divide is deferred: sum of squares (one partial per workgroup), momentum
// update in place if asked for, and the unnormalised bf16 cast, transposed.
template <bool F64>
__global__ void __launch_bounds__(256) sumsq_transpose_kernel(const float* __restrict__ x, int64_t rows, int64_t cols,
                                                              double* __restrict__ partials, MomentumSrc mom,
                                                              uint16_t* __restrict__ raw_out) {
  const int64_t b = blockIdx.y;
  __shared__ double scratch_d[NORM_THREADS / 64];
  __shared__ float tile[64][65];
  const TileWalk w(rows, cols);
  const float* __restrict__ xb = x + b * rows * cols;
  float* __restrict__ mb = mom.buf ? mom.buf + b * rows * cols : nullptr;
  uint16_t* __restrict__ ob = raw_out + b * rows * cols;
  float sf = 0.0f;
  double sd = 0.0;
  for (int64_t t = blockIdx.x; t < w.ntiles; t += gridDim.x) {
    const int64_t r0 = (t / w.tiles_c) * 64, c0 = (t % w.tiles_c) * 64;
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
      const int r = pass * 16 + (threadIdx.x >> 4), c = (threadIdx.x & 15) * 4;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (r0 + r < rows && c0 + c < cols) {
        const int64_t at = (r0 + r) * cols + c0 + c;
        v = stream_load(reinterpret_cast<const float4*>(xb + at));
        if (mb) {
          float4 m = *reinterpret_cast<const float4*>(mb + at);
          m.x = torch_lerp(m.x, v.x, 1.0f - mom.beta);
          m.y = torch_lerp(m.y, v.y, 1.0f - mom.beta);
          m.z = torch_lerp(m.z, v.z, 1.0f - mom.beta);
          m.w = torch_lerp(m.w, v.w, 1.0f - mom.beta);
          *reinterpret_cast<float4*>(mb + at) = m;
          v.x = momentum_direction(v.x, m.x, mom.beta, mom.nesterov);
          v.y = momentum_direction(v.y, m.y, mom.beta, mom.nesterov);
          v.z = momentum_direction(v.z, m.z, mom.beta, mom.nesterov);
          v.w = momentum_direction(v.w, m.w, mom.beta, mom.nesterov);
        }
      }
      if (F64) {
        sd += (double)v.x * (double)v.x + (double)v.y * (double)v.y + (double)v.z * (double)v.z + (double)v.w * (double)v.w;
      } else {
        sf = __builtin_fmaf(v.x, v.x, sf);
        sf = __builtin_fmaf(v.y, v.y, sf);
        sf = __builtin_fmaf(v.z, v.z, sf);
        sf = __builtin_fmaf(v.w, v.w, sf);
      }
      tile[r][c] = v.x;
      tile[r][c + 1] = v.y;
      tile[r][c + 2] = v.z;
      tile[r][c + 3] = v.w;
    }
    __syncthreads();
    store_tile_transposed(tile, ob, rows, cols, r0, c0, 1.0f);
    __syncthreads();
  }
  const double total = block_sum<double>(F64 ? sd : (double)sf, scratch_d);
  if (threadIdx.x == 0) partials[b * gridDim.x + blockIdx.x] = total;
}

// Divide + bf16 cast + transpose.  `xscale` != null: `out` already holds the unnormalised cast; this pass then only
// has work to do for a norm outside the range where the divide may be deferred (see scale_cast_kernel).
__global__ void __launch_bounds__(256) scale_cast_transpose_kernel(const float* __restrict__ x, int64_t rows, int64_t cols,
                                                                   const double* __restrict__ partials, int nparts,
                                                                   float eps, int f64, uint16_t* __restrict__ out,
                                                                   float* __restrict__ dev_norm,
                                                                   float* __restrict__ sumsq_out, MomentumSrc mom,
                                                                   float* __restrict__ xscale) {
  const int64_t b = blockIdx.y;
  __shared__ double scratch_d[NORM_THREADS / 64];
  __shared__ float tile[64][65];
  double s = 0;
  for (int i = threadIdx.x; i < nparts; i += NORM_THREADS) s += partials[b * nparts + i];
  s = block_sum<double>(s, scratch_d);
  const float divisor = f64 ? (float)sqrt(s) : fmaxf(sqrtf((float)s), eps);
  bool deferred = false;
  if (xscale) deferred = divisor >= NORM_DEFER_MIN && divisor <= NORM_DEFER_MAX;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    if (dev_norm) dev_norm[b] = divisor;
    if (sumsq_out) {
      const float ratio = sqrtf((float)s) / divisor;
      sumsq_out[b] = (divisor > 0.0f && ratio == ratio) ? ratio * ratio : 0.0f;
    }
    if (xscale) xscale[b] = deferred ? 1.0f / divisor : 1.0f;
  }
  if (deferred) return;
  const TileWalk w(rows, cols);
  const float* __restrict__ xb = x + b * rows * cols;
  uint16_t* __restrict__ ob = out + b * rows * cols;
  for (int64_t t = blockIdx.x; t < w.ntiles; t += gridDim.x) {
    const int64_t r0 = (t / w.tiles_c) * 64, c0 = (t % w.tiles_c) * 64;
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
      const int r = pass * 16 + (threadIdx.x >> 4), c = (threadIdx.x & 15) * 4;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (r0 + r < rows && c0 + c < cols) {
        v = *reinterpret_cast<const float4*>(xb + (r0 + r) * cols + c0 + c);
        if (mom.buf) {
          const float4 mb = *reinterpret_cast<const float4*>(mom.buf + b * rows * cols + (r0 + r) * cols + c0 + c);
          v.x = momentum_direction(v.x, mb.x, mom.beta, mom.nesterov);
          v.y = momentum_direction(v.y, mb.y, mom.beta, mom.nesterov);
          v.z = momentum_direction(v.z, mb.z, mom.beta, mom.nesterov);
          v.w = momentum_direction(v.w, mb.w, mom.beta, mom.nesterov);
        }
      }
      tile[r][c] = v.x;
      tile[r][c + 1] = v.y;
      tile[r][c + 2] = v.z;
      tile[r][c + 3] = v.w;
    }
    __syncthreads();
    store_tile_transposed(tile, ob, rows, cols, r0, c0, divisor);
    __syncthreads();
  }
}

// out[b][c][r] = in[b][r][c] for float32 (rows x cols) -> (cols x rows); 64 x 64 tiles through LDS.
// With accum != 0 the destination is updated in place: out = accum * out + in^T.
__global__ void __launch_bounds__(256) transpose_f32_kernel(const float* __restrict__ in, int64_t rows, int64_t cols,
                                                            float* __restrict__ out, float accum) {
  const int64_t b = blockIdx.z;
  __shared__ float tile[64][65];
  const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
  const float* __restrict__ ib = in + b * rows * cols;
  float* __restrict__ ob = out + b * rows * cols;
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int r = pass * 16 + (threadIdx.x >> 4), c = (threadIdx.x & 15) * 4;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (r0 + r < rows && c0 + c < cols) v = *reinterpret_cast<const float4*>(ib + (r0 + r) * cols + c0 + c);
    tile[r][c] = v.x;
    tile[r][c + 1] = v.y;
    tile[r][c + 2] = v.z;
    tile[r][c + 3] = v.w;
  }
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int c = pass * 16 + (threadIdx.x >> 4), r = (threadIdx.x & 15) * 4;
    if (c0 + c < cols && r0 + r < rows) {
      f32x4_t v = {tile[r][c], tile[r + 1][c], tile[r + 2][c], tile[r + 3][c]};
      f32x4_t* dst = reinterpret_cast<f32x4_t*>(ob + (c0 + c) * rows + r0 + r);
      if (accum != 0.0f) {
        const f32x4_t old = *dst;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaf(accum, old[e], v[e]);
      }
      *dst = v;
    }
  }
}

static int frob_impl(const float* x, int64_t batch, int64_t numel, float eps, int f64, void* out, int out_bf16,
                     float post_scale, double* partials, float* dev_norm, hipStream_t stream,
                     float* sumsq_out = nullptr, int64_t t_rows = 0, int64_t t_cols = 0,
                     MomentumSrc mom = MomentumSrc{nullptr, 0.0f, 0}, float* xscale = nullptr) {
  if (!x || !out || !partials) return fail(MI_ERR_BAD_ARG, "mi_frob_normalize: null pointer");
  if (batch < 0 || numel < 0) return fail(MI_ERR_BAD_ARG, "mi_frob_normalize: negative extent");
  if (numel % 8) return fail(MI_ERR_UNSUPPORTED_SHAPE, "mi_frob_normalize: numel must be a multiple of 8, got %lld", (long long)numel);
  if (!aligned16(x) || !aligned16(out)) return fail(MI_ERR_UNSUPPORTED_SHAPE, "mi_frob_normalize: pointers must be 16-byte aligned");
  if (batch > 65535) return fail(MI_ERR_UNSUPPORTED_SHAPE, "mi_frob_normalize: batch exceeds 65535");
  if (batch == 0 || numel == 0) return MI_OK;
  const int nb = norm_blocks(numel);
  dim3 grid1(nb, (unsigned)batch), block(NORM_THREADS);
  if (xscale && !out_bf16) return fail(MI_ERR_BAD_ARG, "internal: deferred normalisation needs a bf16 output");
  uint16_t* raw_out = xscale ? static_cast<uint16_t*>(out) : nullptr;
  int nparts = nb;
  if (t_rows > 0 && xscale) {
    // tall input, deferred divide: the first pass already transposes (one partial per workgroup of the tile walk)
    const int64_t ntiles = ((t_rows + 63) / 64) * ((t_cols + 63) / 64);
    nparts = (int)(ntiles < NORM_MAX_BLOCKS ? ntiles : NORM_MAX_BLOCKS);
  }
  // what the two passes cover: the input (and the momentum buffer, updated in place), the cast or the normalised
  // copy, one float64 partial per workgroup of the first pass, one value per matrix of each scalar output
  MI_OTHER_LAUNCH();
  MI_FOOTPRINT("input", x, 4, batch, numel, 1, numel, numel);
  MI_FOOTPRINT("momentum buffer", mom.buf, 4, batch, numel, 1, numel, numel);
  MI_FOOTPRINT("normalised copy", out, out_bf16 ? 2 : 4, batch, numel, 1, numel, numel);
  MI_FOOTPRINT("partial sums of squares", partials, 8, batch, nparts, 1, nparts, nparts);
  MI_FOOTPRINT("norm", dev_norm, 4, 1, 0, 1, batch, batch);
  MI_FOOTPRINT("squared norm of the result", sumsq_out, 4, 1, 0, 1, batch, batch);
  MI_FOOTPRINT("input scale", xscale, 4, 1, 0, 1, batch, batch);
  if (t_rows > 0 && xscale) {
    dim3 gridw((unsigned)nparts, (unsigned)batch);
    if (f64)
      hipLaunchKernelGGL(sumsq_transpose_kernel<true>, gridw, block, 0, stream, x, t_rows, t_cols, partials, mom, raw_out);
    else
      hipLaunchKernelGGL(sumsq_transpose_kernel<false>, gridw, block, 0, stream, x, t_rows, t_cols, partials, mom, raw_out);
  } else if (f64) {
    hipLaunchKernelGGL(sumsq_kernel<true>, grid1, block, 0, stream, x, numel, partials, mom, raw_out);
  } else {
    hipLaunchKernelGGL(sumsq_kernel<false>, grid1, block, 0, stream, x, numel, partials, mom, raw_out);
  }
  if (t_rows > 0) {
    // bf16 output transposed to (t_cols x t_rows)
    const int64_t ntiles = ((t_rows + 63) / 64) * ((t_cols + 63) / 64);
    dim3 gridt((unsigned)(ntiles < 2048 ? ntiles : 2048), (unsigned)batch);
    hipLaunchKernelGGL(scale_cast_transpose_kernel, gridt, block, 0, stream, x, t_rows, t_cols, partials, nparts, eps, f64,
                       static_cast<uint16_t*>(out), dev_norm, sumsq_out, mom, xscale);
    hipError_t et = hipGetLastError();
    if (et != hipSuccess) return fail(MI_ERR_LAUNCH, "mi_frob_normalize launch failed: %s", hipGetErrorString(et));
    return MI_OK;
  }
  int64_t want = (numel / 8 + (int64_t)NORM_THREADS * 4 - 1) / ((int64_t)NORM_THREADS * 4);
  if (want < 1) want = 1;
  // (with a deferred divide nearly every call ends after the norm check: fewer, longer-running workgroups then)
  const int64_t cap = xscale ? 1024 : 4096;
  if (want > cap) want = cap;
  dim3 grid2((unsigned)want, (unsigned)batch);
#define MI_SC(F, B) hipLaunchKernelGGL((scale_cast_kernel<F, B>), grid2, block, 0, stream, x, numel, partials, nb, eps, post_scale, out, dev_norm, sumsq_out, mom, xscale)
  if (f64) {
    if (out_bf16) MI_SC(true, true); else MI_SC(true, false);
  } else {
    if (out_bf16) MI_SC(false, true); else MI_SC(false, false);
  }
#undef MI_SC
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI_ERR_LAUNCH, "mi_frob_normalize launch failed: %s", hipGetErrorString(e));
  return MI_OK;
}

// ---------------------------------------------------------------------------------------------
// Gram matrices of batched short, wide matrices (per-head shapes: 32 x 128 x 4096).  One 128 x 128 output tile
// per matrix cannot fill the chip, so the K range is cut into S slices that run as separate batch entries of a
// plain product (float32 partials), and a second kernel adds the slices in a fixed order, subtracts the
// diagonal shift and mirrors the lower triangle (bitwise symmetric bf16 result).
// ---------------------------------------------------------------------------------------------
// The slice length is fixed (512 columns), so the number of slices -- and with it the order of the float32
// additions -- depends on the shape of one matrix only: a batched call and per-matrix calls agree bit for bit.
static int small_gram_splits(int64_t batch, int64_t m, int64_t n) {
  if (m % 128 != 0 || m > 256 || n % 512 != 0 || n < 1024) return 0;
  const int64_t splits = n / 512;
  if (batch * splits > 65535) return 0;
  return (int)splits;
}

__global__ void __launch_bounds__(256) gram_reduce_kernel(const float* __restrict__ partials, int splits, int m,
                                                          const float* __restrict__ slots_in, int nslots_in,
                                                          float* __restrict__ shift_io, uint16_t* __restrict__ out,
                                                          const float* __restrict__ xscale) {
  const int64_t b = blockIdx.y;
  __shared__ float red[4];
  const float r = xscale ? xscale[b] : 1.0f;
  // diagonal shift of this matrix: ||X||_F^2 / m from the partial sums the previous kernel left
  float part = 0.0f;
  for (int i = threadIdx.x; i < nslots_in; i += 256) part += slots_in[b * nslots_in + i];
  const float shift = block_sum_f32<256>(part, red) / (float)m;
  if (blockIdx.x == 0 && threadIdx.x == 0) shift_io[b] = shift;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= m * m) return;
  const int i = idx / m, j = idx % m;
  if (j > i) return;  // the lower triangle is summed, the upper one is its mirror image
  const float* __restrict__ src = partials + (b * splits) * (int64_t)m * m + idx;
  float acc = 0.0f;
  for (int s = 0; s < splits; ++s) acc += src[(int64_t)s * m * m];
  acc *= r * r;
  if (i == j) acc -= shift;
  const uint16_t h = __builtin_bit_cast(uint16_t, (__bf16)acc);
  uint16_t* __restrict__ ob = out + b * (int64_t)m * m;
  ob[(int64_t)i * m + j] = h;
  ob[(int64_t)j * m + i] = h;
}

// ---------------------------------------------------------------------------------------------
// 128 x 128 matrices (one attention head each): everything between the split-K Gram partials and the B X product
// of a step -- or of a group of two or three steps -- in one launch.  One workgroup per matrix keeps up to four 128 x 128 bf16
// matrices in LDS (32 KB each, 16-byte chunks XOR-swizzled by row so that the 32 rows one fragment read touches
// fall into different banks) and forms
//   D  = r^2 sum_s partial_s - s I                       (what gram_reduce_kernel stores)
//   R1 = c1 D^2 + (b1 + 2 c1 s) D                        single step: the result
//   and for a group of two or three steps the chain R_k, S_k, T'_k, D_{k+1} of SHIFT_GROUP_* (gemm_engine.hpp),
//   whose last S is the result
// with the rounding points of the separate kernels: float32 accumulation, one rounding to bf16 per matrix, the lower
// triangle computed and mirrored.
// ---------------------------------------------------------------------------------------------
static constexpr int CH_M = 128;                       // matrix size served
static constexpr int CH_BYTES = CH_M * CH_M * 2;       // one matrix in LDS
static constexpr int CH_THREADS = 1024;                // 16 wavefronts per workgroup
__device__ __forceinline__ int ch_off(int row, int chunk) { return row * (CH_M * 2) + (((chunk ^ row) & 15) << 4); }
__device__ __forceinline__ int ch_elem(int row, int col) { return ch_off(row, col >> 3) + (col & 7) * 2; }

// Mirror image of an LDS matrix whose lower triangle (diagonal included) is complete: the 16 x 16 blocks on and
// below the diagonal are dealt out to the 16 wavefronts; a wavefront reads a block with the LDS transpose read (16
// lanes fetch 4 rows x 16 columns, 8 bytes each, and lane i receives column i of those four rows) and stores it
// transposed, 8 bytes per lane.  In a diagonal block only what lies right of the diagonal is stored.
__device__ __forceinline__ void chain_mirror(char* mat, int wave, int lane) {
  typedef s16x4_t __attribute__((address_space(3))) * lds_tr_ptr;
  const uint32_t base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)mat;
  const int patch = lane >> 4, i16 = lane & 15;  // rows 4 patch .. + 3 of the block; source lane / destination row
  constexpr int BLOCKS = (CH_M / 16) * (CH_M / 16 + 1) / 2;  // 36
  constexpr int PER_WAVE = (BLOCKS + CH_THREADS / 64 - 1) / (CH_THREADS / 64);  // 3
  uint2 t[PER_WAVE];
  int bi[PER_WAVE], bj[PER_WAVE];
  // (`wave` is uniform: the block indices live in scalar registers; all reads are issued before the first store)
#pragma unroll
  for (int u = 0; u < PER_WAVE; ++u) {
    const int sb = wave + u * (CH_THREADS / 64);
    int r = 0;
#pragma unroll
    for (int c = 1; c < CH_M / 16; ++c) r += (c * (c + 1) / 2 <= sb) ? 1 : 0;  // largest r with r (r + 1) / 2 <= sb
    bi[u] = r;
    bj[u] = sb - r * (r + 1) / 2;
    if (sb < BLOCKS) {
      const int src_row = 16 * bi[u] + 4 * patch + (i16 >> 2), src_col = 16 * bj[u] + 4 * (i16 & 3);
      t[u] = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(uintptr_t)(base + ch_elem(src_row, src_col))));
    }
  }
#pragma unroll
  for (int u = 0; u < PER_WAVE; ++u) {
    if (wave + u * (CH_THREADS / 64) >= BLOCKS) continue;
    // lane i16 holds source rows 16 bi + 4 patch + 0 .. 3 at source column 16 bj + i16
    const int dst_row = 16 * bj[u] + i16, dst_col = 16 * bi[u] + 4 * patch;
    if (bi[u] != bj[u] || dst_col > dst_row) {
      *reinterpret_cast<uint2*>(mat + ch_elem(dst_row, dst_col)) = t[u];
    } else if (dst_col + 3 > dst_row) {
      const uint16_t e[4] = {(uint16_t)(t[u].x & 0xffffu), (uint16_t)(t[u].x >> 16), (uint16_t)(t[u].y & 0xffffu), (uint16_t)(t[u].y >> 16)};
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (dst_col + r > dst_row) *reinterpret_cast<uint16_t*>(mat + ch_elem(dst_row, dst_col + r)) = e[r];
    }
  }
}

// dst = alpha * P Q^T + beta1 * C1 + beta2 * C2 on the lower triangle, mirrored; all operands are LDS matrices.
// Wavefront w of the 16 owns the 32 x 32 block (w / 4, w % 4); the six blocks above the diagonal are only ever
// written as mirror images, so their wavefronts sit the product out.
__device__ __forceinline__ void chain_product(const char* P, const char* Q, const char* C1, const char* C2, char* dst,
                                              float alpha, float beta1, float beta2, int wave, int lane) {
  const int ti = wave >> 2, tj = wave & 3;
  if (tj <= ti) {
    f32x16_t acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.0f;
    const int frow = lane & 31, fk = lane >> 5;
    // the addends do not depend on the product: their reads go out first and arrive behind the MFMAs
    uint2 c1[4], c2[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int m = ti * 32 + frow, n = tj * 32 + 8 * g + 4 * fk;
      c1[g] = *reinterpret_cast<const uint2*>(C1 + ch_elem(m, n));
      c2[g] = C2 != nullptr ? *reinterpret_cast<const uint2*>(C2 + ch_elem(m, n)) : make_uint2(0u, 0u);
    }
#pragma unroll
    for (int q = 0; q < CH_M / 16; ++q) {
      const bf16x8_t fp = *reinterpret_cast<const bf16x8_t*>(P + ch_off(ti * 32 + frow, 2 * q + fk));
      const bf16x8_t fq = *reinterpret_cast<const bf16x8_t*>(Q + ch_off(tj * 32 + frow, 2 * q + fk));
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fq, fp, acc, 0, 0, 0);
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int m = ti * 32 + frow, n = tj * 32 + 8 * g + 4 * fk;
      if (n > m) continue;  // all four columns lie above the diagonal
      f32x4_t v;
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] = alpha * acc[4 * g + r];
      v[0] = __builtin_fmaf(beta1, __uint_as_float(c1[g].x << 16), v[0]);
      v[1] = __builtin_fmaf(beta1, __uint_as_float(c1[g].x & 0xffff0000u), v[1]);
      v[2] = __builtin_fmaf(beta1, __uint_as_float(c1[g].y << 16), v[2]);
      v[3] = __builtin_fmaf(beta1, __uint_as_float(c1[g].y & 0xffff0000u), v[3]);
      if (C2 != nullptr) {
        v[0] = __builtin_fmaf(beta2, __uint_as_float(c2[g].x << 16), v[0]);
        v[1] = __builtin_fmaf(beta2, __uint_as_float(c2[g].x & 0xffff0000u), v[1]);
        v[2] = __builtin_fmaf(beta2, __uint_as_float(c2[g].y << 16), v[2]);
        v[3] = __builtin_fmaf(beta2, __uint_as_float(c2[g].y & 0xffff0000u), v[3]);
      }
      const uint2 h = __builtin_bit_cast(uint2, __builtin_convertvector(v, bf16x4_t));
      if (n + 3 <= m) {
        *reinterpret_cast<uint2*>(dst + ch_elem(m, n)) = h;  // four columns on or below the diagonal
      } else {
        const uint16_t e[4] = {(uint16_t)(h.x & 0xffffu), (uint16_t)(h.x >> 16), (uint16_t)(h.y & 0xffffu), (uint16_t)(h.y >> 16)};
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n + r <= m) *reinterpret_cast<uint16_t*>(dst + ch_elem(m, n + r)) = e[r];
      }
    }
  }
  __syncthreads();  // the lower triangle of dst is complete
  chain_mirror(dst, wave, lane);
  __syncthreads();  // dst is complete, and nobody still reads what the next product overwrites
}

struct ChainArgs {
  const float* partials;  // [batch][splits][128][128] float32
  int splits;
  const float* slots_in;  // partial sums of squares of X, [batch][nslots_in]
  int nslots_in;
  float* shift_io;        // [batch], written
  const float* xscale;    // [batch] or null
  float co[3][3];         // (a, b, c) of the steps of the group
  int group;              // 1, 2 or 3 steps on this Gram matrix
  uint16_t* out;          // [batch][128][128] bf16: the multiplier S_g of X (R_1 for a single step)
};

// One product of the chain: operands, addends and destination as indices of the four LDS matrices (-1: none).
struct ChainOp {
  int p, q, c1, c2, dst;
  float alpha, beta1, beta2;
};
static constexpr int CH_MAX_OPS = 12;  // a group of three steps has 9 products

// 16 wavefronts per workgroup, one per 32 x 32 block of the products; together they stream the float32 partials in
// (the only part that touches HBM; one workgroup per matrix leaves most of the chip idle, so each one needs many
// loads in flight) and the result out.  The products of the chain run as a loop over a small table, so that the code
// of a product exists once and stays in the instruction cache (spelled out nine times, every product was a cold walk
// through new code: 2 us each instead of 1).
__global__ void __launch_bounds__(CH_THREADS) small_chain_kernel(ChainArgs a) {
  __shared__ __align__(16) char chain_lds[4 * CH_BYTES];
  __shared__ float red[CH_THREADS / 64];
  __shared__ ChainOp ops[CH_MAX_OPS];
  __shared__ int nops_lds, result_lds;
  const int64_t b = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: what depends on it alone branches on the scalar unit
  char* B0 = chain_lds;
  // D -> B0.  Only the groups of four columns that start on or left of the diagonal are needed: 33 per pair of rows
  // (p, 127 - p), 2112 in all.  Every thread takes two of them, with all slices (up to 8 at a time) in flight at once;
  // the 64 groups left over are fetched slice by slice by 512 threads, parked in LDS (in a matrix buffer that is
  // still free) and added up, in slice order like the others, by 64 threads.  The shift is summed while the loads fly.
  const float* __restrict__ src = a.partials + b * a.splits * (int64_t)(CH_M * CH_M);
  constexpr int PAIR_GROUPS = CH_M / 4 + 1, LOWER_GROUPS = (CH_M / 2) * PAIR_GROUPS, DEPTH = 8;
  static_assert(LOWER_GROUPS > 2 * CH_THREADS && LOWER_GROUPS - 2 * CH_THREADS <= 64, "two groups per thread and at most 64 left over");
  constexpr int EXTRA = LOWER_GROUPS - 2 * CH_THREADS;
  auto group_of = [](int g, int& i, int& j) {  // g-th needed group -> row i, first column j
    const int pair = g / PAIR_GROUPS, r = g % PAIR_GROUPS, n_lo = pair / 4 + 1;
    i = r < n_lo ? pair : CH_M - 1 - pair;
    j = 4 * (r < n_lo ? r : r - n_lo);
  };
  int gi[3], gj[3];
  group_of(tid, gi[0], gj[0]);
  group_of(tid + CH_THREADS, gi[1], gj[1]);
  group_of(2 * CH_THREADS + (tid < EXTRA ? tid : 0), gi[2], gj[2]);
  int xi, xj;  // the left-over group this thread fetches one slice of
  group_of(2 * CH_THREADS + ((tid >> 3) < EXTRA ? (tid >> 3) : 0), xi, xj);
  f32x4_t* parked = reinterpret_cast<f32x4_t*>(chain_lds + CH_BYTES);  // [EXTRA][DEPTH]
  f32x4_t sum[3];
#pragma unroll
  for (int t = 0; t < 3; ++t) sum[t] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
  float s = 0.0f;
  for (int sp0 = 0; sp0 < a.splits; sp0 += DEPTH) {
    f32x4_t v[2][DEPTH], x = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int u = 0; u < DEPTH; ++u) {
        v[t][u] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        if (sp0 + u < a.splits)
          v[t][u] = *reinterpret_cast<const f32x4_t*>(src + (int64_t)(sp0 + u) * (CH_M * CH_M) + gi[t] * CH_M + gj[t]);
      }
    if ((tid >> 3) < EXTRA && sp0 + (tid & 7) < a.splits)
      x = *reinterpret_cast<const f32x4_t*>(src + (int64_t)(sp0 + (tid & 7)) * (CH_M * CH_M) + xi * CH_M + xj);
    if (sp0 > 0) __syncthreads();  // the parked slices of the previous round have been added
    if ((tid >> 3) < EXTRA) parked[tid] = x;
    if (sp0 == 0) {
      // shift and input scale of this matrix, as gram_reduce_kernel resolves them (its barriers also publish `parked`)
      float part = 0.0f;
      for (int i = tid; i < a.nslots_in; i += CH_THREADS) part += a.slots_in[b * a.nslots_in + i];
      s = block_sum_f32<CH_THREADS>(part, red) / (float)CH_M;
      if (tid == 0) a.shift_io[b] = s;
    } else {
      __syncthreads();
    }
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int u = 0; u < DEPTH; ++u)
        if (sp0 + u < a.splits) sum[t] += v[t][u];
    if (tid < EXTRA) {
#pragma unroll
      for (int u = 0; u < DEPTH; ++u)
        if (sp0 + u < a.splits) sum[2] += parked[tid * DEPTH + u];
    }
  }
  const float r = a.xscale ? a.xscale[b] : 1.0f;
  __syncthreads();  // (the buffer behind `parked` becomes a matrix again)
#pragma unroll
  for (int t = 0; t < 3; ++t) {
    if (t == 2 && tid >= EXTRA) continue;
    const int i = gi[t], j = gj[t];
    f32x4_t d;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      d[e] = sum[t][e] * (r * r);
      if (i == j + e) d[e] -= s;
    }
    const uint2 h = __builtin_bit_cast(uint2, __builtin_convertvector(d, bf16x4_t));
    if (j + 3 <= i) {
      *reinterpret_cast<uint2*>(B0 + ch_elem(i, j)) = h;
    } else {
      const uint16_t e[4] = {(uint16_t)(h.x & 0xffffu), (uint16_t)(h.x >> 16), (uint16_t)(h.y & 0xffffu), (uint16_t)(h.y >> 16)};
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (j + q <= i) *reinterpret_cast<uint16_t*>(B0 + ch_elem(i, j + q)) = e[q];
    }
  }
  // The steps of the group (SHIFT_GROUP_* in gemm_engine.hpp spells out the recursion) as a table of products; D_k
  // stays in matrix 0, the other three are handed out and returned as what they hold dies.
  if (tid == 0) {
    int pool[3] = {1, 2, 3};
    int free_n = 3, n = 0, D = 0, S = -1;
    float sk = s, before = 1.0f;
    for (int k = 0; k < 3 && k < a.group; ++k) {
      const float ak = a.co[k][0], bk = a.co[k][1], ck = a.co[k][2];
      const float e = ak + bk * sk + ck * sk * sk;
      const int R = pool[--free_n];
      ops[n++] = ChainOp{D, D, D, -1, R, ck, bk + 2.0f * ck * sk, 0.0f};  // R_k
      if (k == 0) {
        S = R;
      } else {
        const int Sk = pool[--free_n];
        ops[n++] = ChainOp{R, S, S, R, Sk, 1.0f, e, before};  // S_k
        pool[free_n++] = S;
        S = Sk;
      }
      if (k + 1 < a.group) {
        const int T = pool[--free_n];
        ops[n++] = ChainOp{R, D, D, R, T, 1.0f, e, sk};         // T'_k
        ops[n++] = ChainOp{R, T, T, R, D, 1.0f, e, e * sk};     // D_{k+1} over D_k
        pool[free_n++] = T;
        sk = e * e * sk;
      }
      if (k > 0) pool[free_n++] = R;
      before *= e;
    }
    nops_lds = n;
    result_lds = S;
  }
  __syncthreads();  // the lower triangle of D and the table are complete
  chain_mirror(B0, wave, lane);
  __syncthreads();
  const int nops = nops_lds;
#pragma unroll 1
  for (int o = 0; o < nops; ++o) {
    const ChainOp op = ops[o];
    chain_product(chain_lds + op.p * CH_BYTES, chain_lds + op.q * CH_BYTES, chain_lds + op.c1 * CH_BYTES,
                  op.c2 >= 0 ? chain_lds + op.c2 * CH_BYTES : nullptr, chain_lds + op.dst * CH_BYTES, op.alpha, op.beta1,
                  op.beta2, wave, lane);
  }
  const char* result = chain_lds + result_lds * CH_BYTES;
  uint16_t* __restrict__ ob = a.out + b * (int64_t)(CH_M * CH_M);
  for (int c = tid; c < CH_M * (CH_M / 8); c += CH_THREADS) {
    const int row = c / (CH_M / 8), ch = c % (CH_M / 8);
    *reinterpret_cast<uint4*>(ob + row * CH_M + ch * 8) = *reinterpret_cast<const uint4*>(result + ch_off(row, ch));
  }
}

// Split-K partial Gram matrices: the K range is cut into `splits` slices that run as extra batch entries.
static int small_gram_partials(const uint16_t* X, int64_t batch, int64_t m, int64_t n, int splits, float* partials,
                               hipStream_t stream) {
  GemmParams p{};
  p.P = p.Q = X;
  p.ldp = p.ldq = n;
  p.p_bs = p.q_bs = m * n;
  p.batch_inner = splits;
  p.p_bs2 = p.q_bs2 = n / splits;
  p.Out = partials;
  p.ldo = m;
  p.o_bs = m * m;
  p.M = p.N = (int)m;
  p.K = (int)(n / splits);
  p.alpha = 1.0f;
  p.beta = 0.0f;
  p.out_scale = 1.0f;
  return launch_fast<CfgT128, false, false, MODE_GEMM, true>(p, batch * splits, stream);
}

static int small_gram(const uint16_t* X, int64_t batch, int64_t m, int64_t n, int splits, float* partials,
                      const float* slots_in, int nslots_in, float* shift_io, uint16_t* gram, hipStream_t stream,
                      const float* xscale) {
  int rc = small_gram_partials(X, batch, m, n, splits, partials, stream);
  if (rc != MI_OK) return rc;
  dim3 grid((unsigned)((m * m + 255) / 256), (unsigned)batch), block(256);
  MI_OTHER_LAUNCH();
  MI_FOOTPRINT("Gram partials", partials, 4, batch, splits * m * m, splits, m * m, m * m);
  MI_FOOTPRINT("partial sums read", slots_in, 4, batch, nslots_in, 1, nslots_in, nslots_in);
  MI_FOOTPRINT("shift written", shift_io, 4, 1, 0, 1, batch, batch);
  MI_FOOTPRINT("Gram matrix", gram, 2, batch, m * m, m, m, m);
  MI_FOOTPRINT("input scale read", xscale, 4, 1, 0, 1, batch, batch);
  hipLaunchKernelGGL(gram_reduce_kernel, grid, block, 0, stream, partials, splits, (int)m, slots_in, nslots_in, shift_io, gram, xscale);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI_ERR_LAUNCH, "gram_reduce launch failed: %s", hipGetErrorString(e));
  return MI_OK;
}

// Partials, then everything up to the multiplier of the B X product in one launch (128-row matrices only).
static int small_chain(const uint16_t* X, int64_t batch, int64_t n, int splits, float* partials, const float* slots_in,
                       int nslots_in, float* shift_io, const float* xscale, const float* abc, int group, uint16_t* out,
                       hipStream_t stream, bool have_partials) {
  // (the product that ended the previous group may have left the partials of its result already)
  if (!have_partials) {
    int rc = small_gram_partials(X, batch, CH_M, n, splits, partials, stream);
    if (rc != MI_OK) return rc;
  }
  ChainArgs a{};
  a.partials = partials;
  a.splits = splits;
  a.slots_in = slots_in;
  a.nslots_in = nslots_in;
  a.shift_io = shift_io;
  a.xscale = xscale;
  for (int k = 0; k < group; ++k)
    for (int e = 0; e < 3; ++e) a.co[k][e] = abc[3 * k + e];
  a.group = group;
  a.out = out;
  MI_OTHER_LAUNCH();
  MI_FOOTPRINT("Gram partials", partials, 4, batch, (int64_t)splits * CH_M * CH_M, splits, CH_M * CH_M, CH_M * CH_M);
  MI_FOOTPRINT("partial sums read", slots_in, 4, batch, nslots_in, 1, nslots_in, nslots_in);
  MI_FOOTPRINT("shift written", shift_io, 4, 1, 0, 1, batch, batch);
  MI_FOOTPRINT("input scale read", xscale, 4, 1, 0, 1, batch, batch);
  MI_FOOTPRINT("multiplier of X", out, 2, batch, CH_M * CH_M, CH_M, CH_M, CH_M);
  hipLaunchKernelGGL(small_chain_kernel, dim3((unsigned)batch), dim3(CH_THREADS), 0, stream, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI_ERR_LAUNCH, "small_chain launch failed: %s", hipGetErrorString(e));
  return MI_OK;
}

static size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Tall input iterated as (m x n), m < n: does the last product write the float32 result transposed, straight into the
// output?  (Not on the slab kernel of 128-row matrices.  Option "tall_direct" = 0, read by the workspace query and by
// the call alike: staging copy and transposing pass for every tall input -- A/B runs, tests.)
static bool tall_writes_direct(int64_t m, int64_t n, int gram_splits) {
  return gemm_transposed_out_ok(m, n) && !(gram_splits > 0 && m == CH_M) && opt(OPT_TALL_DIRECT) != 0;
}

struct NsWorkspace {
  size_t x0, x1, a, b, t, d2, partials, norm, slots, shift, xscale, result, gpart, total;
  int gram_splits;  // > 0: split-K Gram path of short, wide batches
  int pairs;        // steps may be taken two at a time on one Gram matrix (two more m x m buffers)
  int64_t max_slots;
};

// Whether consecutive steps share one Gram matrix (see SHIFT_GROUP_* in gemm_engine.hpp): 0 = never, 1 = pairs,
// 2 = pairs, and the first three steps as one group.  A group of g steps trades g - 1 X X^T and g - 1 B X products
// (3 m^2 n multiply-adds each time) for 4 (g - 1) products of m x m matrices, which pays for wide matrices only; on
// a square matrix it would also sit close to the 1e-2 tolerance; below 1024 rows the kernels are launch-bound and a
// group has more launches, except on the split-K Gram path.  Option "ns_pairs": 0 switches grouping off, 1 keeps the
// rule but never takes three steps at once, 2 pairs wherever the kernels allow it (used by the tests to reach the
// pair kernels with small matrices), -1 (default) the rule as described.
static int ns_pairs_enabled(int64_t m, int64_t n, int gram_splits) {
  const int mode = opt(OPT_NS_PAIRS);
  if (mode == 0) return 0;
  if (mode == 2) return 1;
  // (the split-K Gram path serves short matrices at least four times as wide as tall: a group there trades passes
  // over X for tiny products at no more launches)
  if (gram_splits > 0 || (m >= 1024 && n >= 2 * m)) return mode == 1 ? 1 : 2;
  return 0;
}

// Size of the group of steps that starts at step s.  Pairs alternate with single steps (two pairs in a row from
// the start lose accuracy on flat spectra).  Three steps go together only at the very start, where the steps that
// follow damp what the longer chain of m x m products adds, and only if the rounding noise of the first Gram matrix
// is not amplified too much on the way to the third (by (a_1 a_2)^2 in the directions of small singular values:
// 141 for the "simple" coefficients, 260 for "quintic", above 1000 for "polar_express" and "cans").
static int ns_group_size(int mode, const float* abc, int steps, int s, bool want_group) {
  if (!mode || !want_group || s + 1 >= steps) return 1;
  auto quintic = [&](int k) { return abc[3 * k + 2] != 0.0f; };
  if (!quintic(s) || !quintic(s + 1)) return 1;
  if (mode == 2 && s == 0 && steps >= 5 && quintic(2)) {
    const double amp = (double)abc[0] * abc[3];
    if (amp * amp <= 400.0) return 3;
  }
  return 2;
}

static NsWorkspace ns_layout(int64_t batch, int64_t rows, int64_t cols) {
  const int64_t m = rows < cols ? rows : cols;
  NsWorkspace w{};
  size_t off = 0;
  const size_t xbytes = align_up((size_t)batch * rows * cols * 2, 256);
  const size_t gbytes = align_up((size_t)batch * m * m * 2, 256);
  w.x0 = off; off += xbytes;
  w.x1 = off; off += xbytes;
  w.a = off; off += gbytes;
  w.b = off; off += gbytes;
  w.gram_splits = small_gram_splits(batch, m, rows < cols ? cols : rows);
  w.pairs = ns_pairs_enabled(m, rows < cols ? cols : rows, w.gram_splits);
  w.t = off; off += w.pairs ? gbytes : 0;
  w.d2 = off; off += w.pairs ? gbytes : 0;
  w.partials = off; off += align_up((size_t)batch * NORM_MAX_BLOCKS * sizeof(double), 256);
  w.norm = off; off += align_up((size_t)batch * sizeof(float), 256);
  // one float per GEMM workgroup; the smallest tile class (64 x 64) bounds the count
  w.max_slots = ((rows + 63) / 64) * ((cols + 63) / 64);
  w.slots = off; off += align_up((size_t)batch * w.max_slots * sizeof(float), 256);
  w.shift = off; off += align_up((size_t)batch * sizeof(float), 256);
  w.xscale = off; off += align_up((size_t)batch * sizeof(float), 256);
  // tall inputs iterate on the transposed orientation; where the last product cannot write its float32 result
  // transposed, it is staged here before the final transpose into `out`
  w.result = off;
  if (rows > cols && !tall_writes_direct(cols, rows, w.gram_splits)) off += align_up((size_t)batch * rows * cols * sizeof(float), 256);
  // float32 partial Gram matrices of the split-K path
  w.gpart = off;
  off += align_up((size_t)batch * w.gram_splits * m * m * sizeof(float), 256);
  w.total = off;
  return w;
}

// ---------------------------------------------------------------------------------------------
// Built-in scratch of mi_newton_schulz_bf16_noalloc: device memory that belongs to the loaded library itself (one
// copy per GPU, held until the process ends), for callers that cannot allocate a workspace.
// In host code `scratch` is only a handle for the symbol lookup below, never an address to hand to a kernel: each
// device has its own copy at its own address, resolved once per device by hipGetSymbolAddress with that device current.
// ---------------------------------------------------------------------------------------------
static constexpr size_t SCRATCH_BYTES = MI_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];

static constexpr int SCRATCH_MAX_DEVICES = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[SCRATCH_MAX_DEVICES] = {};

// Address of the current device's copy of `scratch` (looked up on the first call on that device).
static int scratch_of_current_device(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(MI_ERR_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= SCRATCH_MAX_DEVICES) return fail(MI_ERR_BAD_ARG, "device index %d is not supported", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr)
      return fail(MI_ERR_LAUNCH, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return MI_OK;
}

}  // namespace mi

using namespace mi;

// Shared body of mi_newton_schulz_bf16 and mi_muon_update_bf16.  `mom.buf` != null: x is the gradient and the
// matrix that is orthogonalised is the momentum direction (the buffer is updated in place on the way).
// `out_accum` != 0: out is updated in place, out = out_accum * out + out_scale * result.
static int ns_impl(const float* x, float* out, int64_t batch, int64_t rows, int64_t cols, const float* abc, int steps,
                   float eps, int accumulate_fp64, float out_scale, void* workspace, size_t workspace_bytes,
                   hipStream_t stream, MomentumSrc mom, float out_accum) {
  if (!x || !out) return fail(MI_ERR_BAD_ARG, "mi_newton_schulz_bf16: null tensor pointer");
  if (batch < 0 || rows < 0 || cols < 0 || steps < 0) return fail(MI_ERR_BAD_ARG, "mi_newton_schulz_bf16: negative argument");
  if (steps > 0 && !abc) return fail(MI_ERR_BAD_ARG, "mi_newton_schulz_bf16: abc is null");
  if (rows % 8 || cols % 8)
    return fail(MI_ERR_UNSUPPORTED_SHAPE, "rows and cols must be multiples of 8, got %lld x %lld", (long long)rows, (long long)cols);
  if (batch == 0 || rows == 0 || cols == 0) return MI_OK;
  // Everything that can be refused is refused here, before the first kernel: the fused optimizer update changes the
  // momentum buffer in its first pass, and an error after that would leave the state half updated.
  if (batch > 65535) return fail(MI_ERR_UNSUPPORTED_SHAPE, "batch %lld exceeds the grid limit 65535", (long long)batch);
  if (!aligned16(x) || !aligned16(out)) return fail(MI_ERR_UNSUPPORTED_SHAPE, "mi_newton_schulz_bf16: tensors must be 16-byte aligned");
  if (rows > (1 << 30) || cols > (1 << 30)) return fail(MI_ERR_UNSUPPORTED_SHAPE, "mi_newton_schulz_bf16: extent too large");
  const NsWorkspace w = ns_layout(batch, rows, cols);
  if (w.max_slots > INT32_MAX) return fail(MI_ERR_UNSUPPORTED_SHAPE, "mi_newton_schulz_bf16: matrix too large");
  if (!workspace || workspace_bytes < w.total)
    return fail(MI_ERR_WORKSPACE, "workspace too small: need %zu bytes, got %zu", w.total, workspace_bytes);
  if (reinterpret_cast<uintptr_t>(workspace) & 255u) return fail(MI_ERR_WORKSPACE, "workspace must be 256-byte aligned");

  char* ws = static_cast<char*>(workspace);
#ifdef MI_HOST_CHECK
  {  // the segments of the workspace as buffers of their own: an access that strays from one into the next is caught
    const size_t at[] = {w.x0, w.x1, w.a, w.b, w.t, w.d2, w.partials, w.norm, w.slots, w.shift, w.xscale, w.result, w.gpart, w.total};
    const char* const names[] = {"ws.x0", "ws.x1", "ws.gram", "ws.poly", "ws.t", "ws.d2", "ws.partials", "ws.norm", "ws.slots",
                                 "ws.shift", "ws.xscale", "ws.result", "ws.gpart"};
    for (int i = 0; i < 13; ++i) host_check::add_range(ws + at[i], at[i + 1] - at[i], names[i]);
  }
#endif
  uint16_t* xbuf[2] = {reinterpret_cast<uint16_t*>(ws + w.x0), reinterpret_cast<uint16_t*>(ws + w.x1)};
  uint16_t* gram = reinterpret_cast<uint16_t*>(ws + w.a);
  uint16_t* poly = reinterpret_cast<uint16_t*>(ws + w.b);
  double* partials = reinterpret_cast<double*>(ws + w.partials);
  float* norm = reinterpret_cast<float*>(ws + w.norm);

  const int64_t numel = rows * cols;
  if (steps == 0) {
    if (mom.buf || out_accum != 0.0f) return fail(MI_ERR_BAD_ARG, "the fused optimizer update needs at least one step");
    return frob_impl(x, batch, numel, eps, accumulate_fp64, out, /*out_bf16=*/0, out_scale, partials, norm, stream);
  }

  float* slots = reinterpret_cast<float*>(ws + w.slots);
  float* shift = reinterpret_cast<float*>(ws + w.shift);
  // The iteration runs on the (m x n) orientation with m <= n, K-contiguous in memory.  A tall input is
  // transposed while it is cast to bf16, and its float32 result is transposed back at the end.
  const int tall = rows > cols;
  const int trans = 0;
  const int64_t m = tall ? cols : rows, n = tall ? rows : cols;
  const int64_t ld = n;
  const int64_t x_bs = numel, g_bs = m * m;
  // (where the last product can write its float32 result transposed, a tall input needs neither the staging copy
  // nor the transposing pass at the end)
  const bool direct_t = tall && tall_writes_direct(m, n, w.gram_splits);
  float* result = (tall && !direct_t) ? reinterpret_cast<float*>(ws + w.result) : out;
  // The input is cast to bf16 by the pass that sums its squares (transposing, if it is tall), and the divide by the
  // norm is folded into the first Gram product and the first B X product: one pass over the float32 input, not two.
  float* xscale = reinterpret_cast<float*>(ws + w.xscale);
  int rc;
  // 128-row matrices whose first group goes through the chain kernel: the input pass also leaves the partial Gram
  // matrices of its bf16 copy (option "head_front" = 0: the general passes and a Gram kernel of its own).
  const bool head_front = w.gram_splits > 0 && m == CH_M && !tall && !accumulate_fp64 && abc[2] != 0.0f &&
                          w.gram_splits == n / 512 && w.gram_splits <= NORM_MAX_BLOCKS && opt(OPT_HEAD_FRONT) != 0 &&
                          head_front_supported(x, batch, n, mom);
  {
    ProfScope prof(PROF_NORMALIZE, stream);
    if (head_front)
      rc = launch_head_front(x, batch, n, eps, mom, xbuf[0], partials, reinterpret_cast<float*>(ws + w.gpart), norm, slots,
                             xscale, stream);
    else
      rc = frob_impl(x, batch, numel, eps, accumulate_fp64, xbuf[0], /*out_bf16=*/1, 1.0f, partials, norm, stream, slots,
                     tall ? rows : 0, tall ? cols : 0, mom, xscale);
  }
  if (rc != MI_OK) return rc;

  int cur = 0;
  int nslots = 1;  // the normalisation kernel left one value per matrix
  bool want_group = true;
  bool have_partials = head_front;  // the partial Gram matrices of xbuf[cur] are in the workspace already
  for (int s = 0; s < steps;) {
    const float a = abc[3 * s], b = abc[3 * s + 1], c = abc[3 * s + 2];
    const int taken = ns_group_size(w.pairs, abc, steps, s, want_group);
    const bool last = (s + taken == steps);
    want_group = taken != 2;  // a pair is followed by a single step; the opening triple may be followed by a pair
    const float* xs = (s == 0) ? xscale : nullptr;  // only the input of the first group is unnormalised
    const uint16_t* mult = gram;
    float alpha = b;
    int apply_mode = SHIFT_APPLY;
    const bool chain = w.gram_splits > 0 && m == CH_M && c != 0.0f;
    if (chain) {
      // 128-row matrices: Gram partials, then one launch per matrix for everything up to the multiplier of X
      {
        ProfScope prof(PROF_GRAM, stream);
        rc = small_chain(xbuf[cur], batch, n, w.gram_splits, reinterpret_cast<float*>(ws + w.gpart), slots, nslots, shift, xs,
                         abc + 3 * s, taken, poly, stream, have_partials);
      }
      if (rc != MI_OK) return rc;
      mult = poly;
      alpha = 1.0f;
      if (taken > 1) apply_mode = SHIFT_GROUP_APPLY;
    } else {
      // A' = X X^T - s I  (s = ||X||_F^2 / m from the partial sums the previous kernel left)
      ShiftArgs sh_gram{SHIFT_GRAM, b, c, slots, nslots, shift, nullptr};
      sh_gram.xscale = xs;
      {
        ProfScope prof(PROF_GRAM, stream);
        if (w.gram_splits > 0)
          rc = small_gram(xbuf[cur], batch, m, n, w.gram_splits, reinterpret_cast<float*>(ws + w.gpart), slots, nslots, shift,
                          gram, stream, xs);
        else
          rc = syrk_impl(xbuf[cur], batch, m, n, x_bs, ld, trans, nullptr, 0, m, 1.0f, 0.0f, gram, g_bs, m, 0, stream, &sh_gram);
      }
      if (rc != MI_OK) return rc;
      if (taken == 1) {
        if (c != 0.0f) {
          // B' = c A'^2 + (b + 2 c s) A'
          ShiftArgs sh_poly{SHIFT_POLY, b, c, nullptr, 0, shift, nullptr};
          {
            ProfScope prof(PROF_POLY, stream);
            rc = syrk_impl(gram, batch, m, m, g_bs, m, 0, gram, g_bs, m, c, b, poly, g_bs, m, 0, stream, &sh_poly);
          }
          if (rc != MI_OK) return rc;
          mult = poly;
          alpha = 1.0f;
        }
      } else {
        // Several steps on this Gram matrix: products of commuting symmetric m x m matrices (SHIFT_GROUP_* in
        // gemm_engine.hpp; the host coefficient 1 of each addend is replaced on the device, where the shift is
        // known).  Four buffers go round: D_k stays in `gram`, the others are handed out and returned as the
        // matrices they hold die.
        uint16_t* pool[3] = {poly, reinterpret_cast<uint16_t*>(ws + w.t), reinterpret_cast<uint16_t*>(ws + w.d2)};
        int free_n = 3;
        auto take = [&]() { return pool[--free_n]; };
        auto give = [&](uint16_t* buf) { pool[free_n++] = buf; };
        auto product = [&](int mode, int stage, const uint16_t* left, const uint16_t* right, const uint16_t* add2, float al,
                           uint16_t* dst) {
          ShiftArgs sh{mode, b, c, nullptr, 0, shift, nullptr};
          sh.group_abc = abc + 3 * s;
          sh.group_size = taken;
          sh.stage = stage;
          ProfScope prof(PROF_POLY, stream);
          return syrk_impl(left, batch, m, m, g_bs, m, 0, right, g_bs, m, al, 1.0f, dst, g_bs, m, 0, stream, &sh,
                           right == left ? nullptr : right, add2);
        };
        uint16_t* D = gram;
        uint16_t* S = nullptr;  // S_{k-1}
        for (int k = 0; k < taken; ++k) {
          // R_k = c_k D_k^2 + (b_k + 2 c_k s_k) D_k
          uint16_t* R = take();
          if ((rc = product(SHIFT_GROUP_POLY, k, D, D, nullptr, abc[3 * (s + k) + 2], R)) != MI_OK) return rc;
          if (k == 0) {
            S = R;  // S_1 = R_1
          } else {
            // S_k = R_k S_{k-1} + e_k S_{k-1} + alpha_{k-1} R_k
            uint16_t* Sk = take();
            if ((rc = product(SHIFT_GROUP_Q, k, R, S, R, 1.0f, Sk)) != MI_OK) return rc;
            give(S);
            S = Sk;
          }
          if (k + 1 < taken) {
            // T'_k = R_k D_k + e_k D_k + s_k R_k, then D_{k+1} = R_k T'_k + e_k T'_k + e_k s_k R_k over D_k
            uint16_t* T = take();
            if ((rc = product(SHIFT_GROUP_T, k, R, D, R, 1.0f, T)) != MI_OK) return rc;
            if ((rc = product(SHIFT_GROUP_A, k, R, T, R, 1.0f, D)) != MI_OK) return rc;
            give(T);
          }
          if (k > 0) give(R);  // (R_1 lives on as S_1)
        }
        mult = S;
        alpha = 1.0f;
        apply_mode = SHIFT_GROUP_APPLY;
      }
    }
    // X' = (a + b s + c s^2) X + B' X      (cubic: (a + b s) X + b A' X;  pair: e1 e2 X + S X)
    void* dst = last ? static_cast<void*>(result) : static_cast<void*>(xbuf[cur ^ 1]);
    ShiftArgs sh_apply{apply_mode, b, c, nullptr, 0, shift, last ? nullptr : slots};
    sh_apply.group_abc = abc + 3 * s;
    sh_apply.group_size = taken;
    sh_apply.stage = taken - 1;
    sh_apply.xscale = xs;
    sh_apply.slot_capacity = (int)w.max_slots;
    {
      ProfScope prof(PROF_APPLY, stream);
      bool head_used = false;
      const bool write_t = last && direct_t;
      rc = gemm_axpy_impl(mult, g_bs, m, xbuf[cur], x_bs, ld, trans, dst, x_bs, write_t ? m : ld, batch, m, n, alpha,
                          taken > 1 ? 1.0f : a, last ? 1 : 0, last ? out_scale : 1.0f, stream, &sh_apply,
                          (last && (!tall || direct_t)) ? out_accum : 0.0f, chain ? w.gram_splits : 0,
                          reinterpret_cast<float*>(ws + w.gpart), &head_used, write_t ? 1 : 0);
      have_partials = head_used && !last;
    }
    if (rc != MI_OK) return rc;
    nslots = g_last_launch.tiles;
    cur ^= 1;
    s += taken;
  }
  if (tall && !direct_t) {
    ProfScope prof(PROF_NORMALIZE, stream);
    dim3 gridt((unsigned)((n + 63) / 64), (unsigned)((m + 63) / 64), (unsigned)batch), blockt(256);
    MI_OTHER_LAUNCH();
    MI_FOOTPRINT("staged result", result, 4, batch, m * n, m, n, n);
    MI_FOOTPRINT("result, transposed back", out, 4, batch, m * n, n, m, m);
    hipLaunchKernelGGL(transpose_f32_kernel, gridt, blockt, 0, stream, result, m, n, out, out_accum);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(MI_ERR_LAUNCH, "transpose launch failed: %s", hipGetErrorString(e));
  }
  return MI_OK;
}


#pragma GCC visibility push(default)
extern "C" {

int mi_version(void) { return 200; }

const char* mi_last_error(void) { return g_last_error.c_str(); }

int mi_syrk_bf16(const void* A, int64_t batch, int64_t n, int64_t k, int64_t a_batch_stride, int64_t a_ld, int a_trans,
                 const void* C, int64_t c_batch_stride, int64_t c_ld, float alpha, float beta, void* D,
                 int64_t d_batch_stride, int64_t d_ld, int skip_upper, void* stream) {
  return syrk_impl(A, batch, n, k, a_batch_stride, a_ld, a_trans, C, c_batch_stride, c_ld, alpha, beta, D,
                   d_batch_stride, d_ld, skip_upper, static_cast<hipStream_t>(stream));
}

size_t mi_syrk_workspace_bytes(int64_t batch, int64_t n, int64_t k, int a_trans) {
  if (batch <= 0 || n <= 0 || k <= 0 || n % 8 || k % 8) return 0;
  StreamKPlan plan;
  const size_t copy = a_trans ? transposed_copy_bytes(n, batch, k) : 0;
  const bool contiguous = !a_trans || copy > 0;
  return copy + (streamk_wanted(n, batch, k, !contiguous, &plan) ? streamk_workspace_bytes(plan) : 0);
}

int mi_syrk_bf16_ws(const void* A, int64_t batch, int64_t n, int64_t k, int64_t a_batch_stride, int64_t a_ld, int a_trans,
                    const void* C, int64_t c_batch_stride, int64_t c_ld, float alpha, float beta, void* D,
                    int64_t d_batch_stride, int64_t d_ld, int skip_upper, void* workspace, size_t workspace_bytes,
                    void* stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  // every argument is checked before the transposing copy below: an invalid call launches nothing
  if (int rc = syrk_validate(A, batch, n, k, a_batch_stride, a_ld, a_trans, C, c_batch_stride, c_ld, beta, D, d_batch_stride, d_ld))
    return rc;
  if (a_trans && workspace && batch > 0 && n > 0 && k > 0 && !(reinterpret_cast<uintptr_t>(workspace) & 255u)) {
    const size_t copy = transposed_copy_bytes(n, batch, k);
    if (copy > 0 && workspace_bytes >= copy && n < (1 << 30) && k < (1 << 30) && batch <= 65535) {
      // the operand, K-contiguous, in the first part of the workspace; the rest serves the product itself
      uint16_t* At = static_cast<uint16_t*>(workspace);
      dim3 grid((unsigned)((n + 63) / 64), (unsigned)((k + 63) / 64), (unsigned)batch);
      MI_OTHER_LAUNCH();
      MI_FOOTPRINT("operand stored as K rows", A, 2, batch, a_batch_stride, k, a_ld, n);
      MI_FOOTPRINT("operand copy, K-contiguous", At, 2, batch, n * k, n, k, k);
      hipLaunchKernelGGL(transpose_bf16_kernel, grid, dim3(256), 0, st, static_cast<const uint16_t*>(A), a_batch_stride, a_ld, At,
                         n * k, k, (int)n, (int)k);
      hipError_t e = hipGetLastError();
      if (e != hipSuccess) return fail(MI_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
      return syrk_impl(At, batch, n, k, n * k, k, 0, C, c_batch_stride, c_ld, alpha, beta, D, d_batch_stride, d_ld, skip_upper,
                       st, nullptr, nullptr, nullptr, static_cast<char*>(workspace) + copy, workspace_bytes - copy);
    }
  }
  return syrk_impl(A, batch, n, k, a_batch_stride, a_ld, a_trans, C, c_batch_stride, c_ld, alpha, beta, D,
                   d_batch_stride, d_ld, skip_upper, st, nullptr, nullptr, nullptr, workspace, workspace_bytes);
}

int mi_gemm_axpy_bf16(const void* Bm, int64_t b_batch_stride, int64_t b_ld, const void* X,
                      int64_t x_batch_stride, int64_t x_ld, int x_trans, void* Xout, int64_t o_batch_stride,
                      int64_t o_ld, int64_t batch, int64_t m, int64_t n, float alpha, float beta, int out_fp32,
                      float out_scale, void* stream) {
  return gemm_axpy_impl(Bm, b_batch_stride, b_ld, X, x_batch_stride, x_ld, x_trans, Xout, o_batch_stride,
                        o_ld, batch, m, n, alpha, beta, out_fp32, out_scale, static_cast<hipStream_t>(stream));
}

size_t mi_frob_partials_len(int64_t batch, int64_t numel) {
  (void)numel;
  return (size_t)(batch < 0 ? 0 : batch) * NORM_MAX_BLOCKS;
}

int mi_frob_normalize(const float* x, int64_t batch, int64_t numel, float eps, int accumulate_fp64, void* out,
                      int out_bf16, double* partials, float* dev_norm, void* stream) {
  return frob_impl(x, batch, numel, eps, accumulate_fp64, out, out_bf16, 1.0f, partials, dev_norm,
                   static_cast<hipStream_t>(stream));
}

int mi_profile_begin(void) {
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  for (auto& sp : g_prof_spans) {
    (void)hipEventDestroy(sp.start);
    (void)hipEventDestroy(sp.stop);
  }
  g_prof_spans.clear();
  g_prof_on = true;
  return MI_OK;
}

int mi_profile_end(float* ms_by_kind, int* launches_by_kind) {
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  g_prof_on = false;
  if (!ms_by_kind || !launches_by_kind) return fail(MI_ERR_BAD_ARG, "mi_profile_end: null output");
  for (int k = 0; k < PROF_KINDS; ++k) {
    ms_by_kind[k] = 0.0f;
    launches_by_kind[k] = 0;
  }
  int rc = MI_OK;
  for (auto& sp : g_prof_spans) {
    float ms = 0.0f;
    if (hipEventSynchronize(sp.stop) != hipSuccess || hipEventElapsedTime(&ms, sp.start, sp.stop) != hipSuccess) {
      rc = fail(MI_ERR_LAUNCH, "mi_profile_end: event query failed");
    } else {
      ms_by_kind[sp.kind] += ms;
      launches_by_kind[sp.kind] += 1;
    }
    (void)hipEventDestroy(sp.start);
    (void)hipEventDestroy(sp.stop);
  }
  g_prof_spans.clear();
  return rc;
}

size_t mi_newton_schulz_workspace_bytes(int64_t batch, int64_t rows, int64_t cols) {
  if (batch <= 0 || rows <= 0 || cols <= 0) return 0;
  return ns_layout(batch, rows, cols).total;
}

int mi_newton_schulz_schedule(int64_t batch, int64_t rows, int64_t cols, const float* abc, int steps, int* groups,
                              int max_groups) {
  if (batch <= 0 || rows <= 0 || cols <= 0 || steps < 0 || (steps > 0 && !abc) || !groups || max_groups < 0)
    return fail(MI_ERR_BAD_ARG, "mi_newton_schulz_schedule: bad argument");
  const NsWorkspace w = ns_layout(batch, rows, cols);
  int count = 0;
  bool want_group = true;
  for (int s = 0; s < steps;) {
    const int taken = ns_group_size(w.pairs, abc, steps, s, want_group);
    want_group = taken != 2;
    if (count < max_groups) groups[count] = taken;
    ++count;
    s += taken;
  }
  return count;
}

int mi_newton_schulz_bf16(const float* x, float* out, int64_t batch, int64_t rows, int64_t cols, const float* abc,
                          int steps, float eps, int accumulate_fp64, float out_scale, void* workspace,
                          size_t workspace_bytes, void* stream) {
  return ns_impl(x, out, batch, rows, cols, abc, steps, eps, accumulate_fp64, out_scale, workspace, workspace_bytes,
                 static_cast<hipStream_t>(stream), MomentumSrc{nullptr, 0.0f, 0}, 0.0f);
}

int mi_newton_schulz_bf16_noalloc(const float* x, float* out, int64_t batch, int64_t rows, int64_t cols, const float* abc,
                                  int steps, float eps, int accumulate_fp64, float out_scale, void* stream) {
  if (batch < 0 || rows < 0 || cols < 0) return fail(MI_ERR_BAD_ARG, "mi_newton_schulz_bf16_noalloc: negative argument");
  if (batch == 0 || rows == 0 || cols == 0) return MI_OK;
  const size_t need = ns_layout(batch, rows, cols).total;
  if (need > SCRATCH_BYTES)
    return fail(MI_ERR_WORKSPACE, "mi_newton_schulz_bf16_noalloc: this call needs %zu bytes of scratch, the built-in buffer has %zu", need,
                SCRATCH_BYTES);
  void* ws = nullptr;
  if (int rc = scratch_of_current_device(&ws)) return rc;
  return ns_impl(x, out, batch, rows, cols, abc, steps, eps, accumulate_fp64, out_scale, ws, SCRATCH_BYTES,
                 static_cast<hipStream_t>(stream), MomentumSrc{nullptr, 0.0f, 0}, 0.0f);
}

int mi_muon_update_bf16(float* param, const float* grad, float* momentum, int64_t batch, int64_t rows, int64_t cols,
                        float beta, int nesterov, float param_decay, float update_scale, const float* abc, int steps,
                        float eps, int accumulate_fp64, void* workspace, size_t workspace_bytes, void* stream) {
  if (!param || !grad || !momentum) return fail(MI_ERR_BAD_ARG, "mi_muon_update_bf16: null tensor pointer");
  if (steps < 1) return fail(MI_ERR_BAD_ARG, "mi_muon_update_bf16: steps must be at least 1");
  if (param_decay == 0.0f) return fail(MI_ERR_BAD_ARG, "mi_muon_update_bf16: param_decay must not be 0");
  if (!aligned16(param) || !aligned16(grad) || !aligned16(momentum))
    return fail(MI_ERR_UNSUPPORTED_SHAPE, "mi_muon_update_bf16: pointers must be 16-byte aligned");
  return ns_impl(grad, param, batch, rows, cols, abc, steps, eps, accumulate_fp64, update_scale, workspace,
                 workspace_bytes, static_cast<hipStream_t>(stream), MomentumSrc{momentum, beta, nesterov ? 1 : 0},
                 param_decay);
}

int mi_set_option(const char* name, int value) {
  const int i = opt_index(name);
  if (i < 0) return fail(MI_ERR_BAD_ARG, "mi_set_option: unknown option '%s'", name ? name : "(null)");
  if (value < OPT_TABLE[i].lo || value > OPT_TABLE[i].hi)
    return fail(MI_ERR_BAD_ARG, "mi_set_option: %s takes %d .. %d, got %d", name, OPT_TABLE[i].lo, OPT_TABLE[i].hi, value);
  opt_init();
  g_opt[i].store(value, std::memory_order_relaxed);
  return MI_OK;
}

int mi_get_option(const char* name, int* value) {
  const int i = opt_index(name);
  if (i < 0 || !value) return fail(MI_ERR_BAD_ARG, "mi_get_option: unknown option '%s' or null output", name ? name : "(null)");
  *value = opt(static_cast<Opt>(i));
  return MI_OK;
}

int mi_debug_last_launch(int* tiles, int* tile_m, int* tile_n, int* fast) {
  if (tiles) *tiles = g_last_launch.tiles;
  if (tile_m) *tile_m = g_last_launch.tile_m;
  if (tile_n) *tile_n = g_last_launch.tile_n;
  if (fast) *fast = g_last_launch.fast;
  return MI_OK;
}

}  // extern "C"
#pragma GCC visibility pop
