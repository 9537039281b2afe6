// bf16 MFMA tile engine for gfx950 (MI355X): OUT[M x N] = epilogue( sum_k P[m][k] * Q[n][k] ).
//
// One template covers the three products of a Newton-Schulz step:
//   SYRK mode : P == Q, only lower-triangle tiles are launched, results are mirrored on store
//   GEMM mode : OUT = beta * Cin + alpha * acc  (the AXPY of X' = a X + B X lives in the epilogue)
// Each operand is either "K-contiguous" (element (r, k) at r*ld + k) or "K-strided"
// (element (r, k) at k*ld + r); K-strided tiles are transposed in registers (v_perm_b32 on 8x8
// blocks) on their way to LDS, so the MFMA fragment reads are always 16-byte ds_read_b128.
//
// Wavefront = 64 lanes; MFMA = v_mfma_f32_32x32x16_bf16.  Fragment/accumulator mapping used here:
//   A operand (32 x 16): lane l supplies row (l % 32), k = 8*(l / 32) .. +7
//   B operand (16 x 32): lane l supplies col (l % 32), k = 8*(l / 32) .. +7
//   D (32 x 32)        : lane l holds col (l % 32); acc[4*g + r] is row 8*g + 4*(l / 32) + r
// The Q fragment is passed as the A operand and the P fragment as the B operand, so a lane ends up
// holding one output row (P index) and groups of 4 consecutive output columns (Q index).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

enum { MODE_SYRK = 0, MODE_GEMM = 1 };

struct GemmParams {
  const uint16_t* P;
  const uint16_t* Q;
  int64_t ldp, ldq, p_bs, q_bs;  // leading dims / batch strides in elements
  // Two-level batch of the operands (fast kernel only): batch entry y reads P at (y / batch_inner) * p_bs +
  // (y % batch_inner) * p_bs2, likewise Q.  batch_inner <= 1 means the plain one-level batch.
  int batch_inner;
  int64_t p_bs2, q_bs2;
  const uint16_t* Cin;           // bf16, indexed like OUT; may be null when beta == 0
  int64_t ldc, c_bs;
  const uint16_t* Cin2;          // SYRK mode, bf16 output: optional second addend, same layout as Cin
  void* Out;                     // bf16 or float32, row-major (M x N)
  int64_t ldo, o_bs;
  int M, N, K;
  float alpha, beta, out_scale;
  float beta2;                   // coefficient of Cin2
  float out_accum;               // float32 output only: Out = out_accum * Out + out_scale * value (0: plain store)
  // float32 output of a GEMM-mode product through the fast kernel's staged epilogue only: Out holds the transposed
  // result, element (m, n) at Out[n * ldo + m] (ldo >= M).  Every other kernel is refused by its launcher.
  int out_transposed;
  int tiles_m, tiles_n;
  int skip_upper;
  // Diagonal-shift bookkeeping of the fused Newton-Schulz driver (all null / 0 for plain calls).
  // The Gram matrix is stored as A' = A - s I with s ~ tr(A)/M, so that bf16 rounding acts on the small
  // deviations of the diagonal instead of on its O(1) magnitude; the identity part is folded back into
  // the epilogue scalars of the two kernels that consume A', which keeps the algebra exact for any s.
  int shift_mode;            // SHIFT_*
  float ca, cb, cc;          // step coefficients a, b, c (host values)
  float co[3][3];            // SHIFT_GROUP_*: (a, b, c) of up to three steps that share one Gram matrix
  int stage;                 // SHIFT_GROUP_*: which of them this launch belongs to (0-based)
  const float* slots_in;     // SHIFT_GRAM: per-tile partial sums of squares of X, [batch][nslots_in]
  int nslots_in;
  float* shift_io;           // [batch]: written by SHIFT_GRAM, read by SHIFT_POLY / SHIFT_APPLY
  // Fused driver, first group of steps only: X is held unnormalised (bf16 of the input) and xscale[batch] =
  // 1 / ||x||_F is applied where X enters a product: squared in SHIFT_GRAM, once in the apply modes.  Null: 1.
  const float* xscale;
  float* slots_out;          // GEMM mode: per-workgroup sum of squares of the output,
  int slot_stride, slot_base;  //   at slots_out[batch * slot_stride + slot_base + blockIdx.x]
  int slot_capacity;         // host side only: floats reserved per batch entry behind slots_out (0: not checked)
  // Lower-triangle launches of the fast kernel number their tiles through the whole batch (tile = batch entry *
  // tiles per matrix + position in the blocked triangular order) on a one-dimensional grid: tiles [0, lin_tiles) in
  // rounds of lin_g workgroups (what the chip holds at once, a multiple of 8), the rest in a last, partial round
  // shared evenly between the XCDs.  Filled in by the launcher.
  int lin_tiles, lin_g;
  // Split-tail launches (see gemm_fast_kernel): the sk_rem tiles from lin_tiles on are split along K between
  // sk_splits workgroups each, sk_tpx left-over tiles per XCD; one float32 accumulator image per (split, tile).
  int sk_rem, sk_splits, sk_tpx;
  float* sk_partials;
};

// Consecutive steps can share one Gram matrix, because every factor involved is a polynomial of it and they all
// commute.  With A_k = s_k I + D_k (D_k stored), step k = (a_k, b_k, c_k), q_k = e_k I + R_k its multiplier and
// Q_k = q_k ... q_1 = alpha_k I + S_k the accumulated one (alpha_k = e_1 ... e_k, S_1 = R_1):
//   R_k  = c_k D_k^2 + (b_k + 2 c_k s_k) D_k,   e_k = a_k + b_k s_k + c_k s_k^2                [SHIFT_GROUP_POLY]
//   S_k  = R_k S_{k-1} + e_k S_{k-1} + alpha_{k-1} R_k                          (k > 1)        [SHIFT_GROUP_Q]
//   T'_k = R_k D_k + e_k D_k + s_k R_k                           (q_k A_k minus its identity)  [SHIFT_GROUP_T]
//   D_{k+1} = R_k T'_k + e_k T'_k + e_k s_k R_k,  s_{k+1} = e_k^2 s_k     (A_{k+1} = q_k^2 A_k) [SHIFT_GROUP_A]
//   X' = alpha_g X + S_g X  after the last step g of the group                                 [SHIFT_GROUP_APPLY]
// A group of g steps costs one X X^T, one B X and 4 g - 3 products of m x m matrices instead of g of each.
enum {
  SHIFT_NONE = 0, SHIFT_GRAM = 1, SHIFT_POLY = 2, SHIFT_APPLY = 3,
  SHIFT_GROUP_POLY = 4, SHIFT_GROUP_T = 5, SHIFT_GROUP_A = 6, SHIFT_GROUP_Q = 7, SHIFT_GROUP_APPLY = 8
};

// Byte offset of 16-byte chunk `chunk` of row `row` in an LDS tile whose rows hold BK bf16 values.
// The XOR swizzle spreads the 16 rows that one quarter-wave reads (same chunk, consecutive rows)
// over all LDS banks, and keeps row-contiguous writes conflict free.
template <int BK>
__device__ __forceinline__ int lds_off(int row, int chunk) {
  constexpr int CPR = BK / 8;
  return row * (BK * 2) + (((chunk ^ (row >> 1) ^ (row >> 3)) & (CPR - 1)) << 4);
}

// Linear lower-triangle tile id -> (ti, tj) with tj <= ti.  ti = floor((sqrt(8 pid + 1) - 1) / 2),
// fixed up with integer arithmetic so float rounding can never produce tj > ti.
__device__ __forceinline__ void tri_decode(int pid, int& ti, int& tj) {
  int t = (int)((sqrtf(8.0f * (float)pid + 1.0f) - 1.0f) * 0.5f);
  while ((t + 1) * (t + 2) / 2 <= pid) ++t;
  while (t * (t + 1) / 2 > pid) --t;
  ti = t;
  tj = pid - t * (t + 1) / 2;
}

// Locality-preserving enumeration of the lower-triangle tiles for the XCD-aware SYRK launch.
// The triangle is cut into block-rows of TRI_BLOCK tile rows; inside a block-row the full
// TRI_BLOCK-wide rectangles come first (row-major inside each), then the triangular block on the
// diagonal.  Consecutive sequence numbers therefore stay inside a ~TRI_BLOCK x TRI_BLOCK block that
// touches only ~2 TRI_BLOCK operand panels.  `s` must be < T (T + 1) / 2.
constexpr int TRI_BLOCK = 6;
__device__ __host__ inline void tri_block_decode(int s, int T, int& ti, int& tj) {
  // block-row: the plain row-major row of s tells which band of TRI_BLOCK rows s falls into
  int r = 0;
#if defined(__HIP_DEVICE_COMPILE__)
  r = (int)((sqrtf(8.0f * (float)s + 1.0f) - 1.0f) * 0.5f);
#else
  while ((r + 1) * (r + 2) / 2 <= s) ++r;
#endif
  while ((r + 1) * (r + 2) / 2 <= s) ++r;
  while (r * (r + 1) / 2 > s) --r;
  const int bi = r / TRI_BLOCK;
  const int row0 = bi * TRI_BLOCK;
  const int h = (T - row0) < TRI_BLOCK ? (T - row0) : TRI_BLOCK;  // rows in this block-row
  int u = s - row0 * (row0 + 1) / 2;                               // index inside the block-row
  const int rect = h * TRI_BLOCK;                                  // tiles per full rectangle
  if (u < bi * rect) {
    const int bj = u / rect, v = u % rect;
    ti = row0 + v / TRI_BLOCK;
    tj = bj * TRI_BLOCK + v % TRI_BLOCK;
    return;
  }
  u -= bi * rect;  // triangular block on the diagonal: plain row-major triangle
  int lr = 0;
  while ((lr + 1) * (lr + 2) / 2 <= u) ++lr;
  ti = row0 + lr;
  tj = row0 + (u - lr * (lr + 1) / 2);
}

__device__ __forceinline__ uint32_t dword_of(const uint4& v, int c) {
  return c == 0 ? v.x : (c == 1 ? v.y : (c == 2 ? v.z : v.w));
}

// ---------------------------------------------------------------------------------------------
// Global -> register -> LDS tile loaders.  ROWS x BK bf16 tile, NT threads.
// ---------------------------------------------------------------------------------------------
template <int ROWS, int BK, int NT, bool KS>
struct TileLoader;

// K-contiguous source: 16-byte chunks copied straight through.
template <int ROWS, int BK, int NT>
struct TileLoader<ROWS, BK, NT, false> {
  static constexpr int CPR = BK / 8;
  static constexpr int NCH = (ROWS * CPR + NT - 1) / NT;
  uint4 r[NCH];

  __device__ __forceinline__ void load(const uint16_t* __restrict__ base, int64_t ld, int row0, int k0, int R,
                                       int K, int tid) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      int ch = tid + i * NT;
      int row = ch / CPR, kc = ch % CPR;
      int gr = row0 + row, gk = k0 + kc * 8;
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (ch < ROWS * CPR && gr < R && gk < K) v = *reinterpret_cast<const uint4*>(base + (int64_t)gr * ld + gk);
      r[i] = v;
    }
  }
  __device__ __forceinline__ void store(char* lds, int tid) const {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      int ch = tid + i * NT;
      int row = ch / CPR, kc = ch % CPR;
      if (ch < ROWS * CPR) *reinterpret_cast<uint4*>(lds + lds_off<BK>(row, kc)) = r[i];
    }
  }
};

// K-strided source: each thread owns 8(k) x 8(rows) blocks, transposes them in registers.
template <int ROWS, int BK, int NT>
struct TileLoader<ROWS, BK, NT, true> {
  static constexpr int KB = BK / 8;
  static constexpr int NBLK = (ROWS / 8) * KB;
  static constexpr int NB = (NBLK + NT - 1) / NT;
  uint4 r[NB][8];

  __device__ __forceinline__ static void decode(int idx, int& rb, int& kb) {
    // 8 consecutive lanes walk along the contiguous (row) dimension: 128-byte global segments.
    int rb_lo = idx & 7;
    kb = (idx >> 3) % KB;
    int rb_hi = (idx >> 3) / KB;
    rb = rb_hi * 8 + rb_lo;
  }
  __device__ __forceinline__ void load(const uint16_t* __restrict__ base, int64_t ld, int row0, int k0, int R,
                                       int K, int tid) {
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      int rb, kb;
      decode(tid + i * NT, rb, kb);
      int gr = row0 + rb * 8;
      bool ok = (tid + i * NT) < NBLK && gr < R;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        int gk = k0 + kb * 8 + e;
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (ok && gk < K) v = *reinterpret_cast<const uint4*>(base + (int64_t)gk * ld + gr);
        r[i][e] = v;
      }
    }
  }
  __device__ __forceinline__ void store(char* lds, int tid) const {
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      int rb, kb;
      decode(tid + i * NT, rb, kb);
      if ((tid + i * NT) >= NBLK) continue;
      // r[i][e] dword c = (x[k=e][row 2c], x[k=e][row 2c+1]); output chunk for row j = x[k=0..7][row j].
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        uint32_t lo[4], hi[4];
#pragma unroll
        for (int pr = 0; pr < 4; ++pr) {
          uint32_t ka = dword_of(r[i][2 * pr], c);
          uint32_t kbv = dword_of(r[i][2 * pr + 1], c);
          lo[pr] = __builtin_amdgcn_perm(kbv, ka, 0x05040100u);  // (ka.lo16, kb.lo16)
          hi[pr] = __builtin_amdgcn_perm(kbv, ka, 0x07060302u);  // (ka.hi16, kb.hi16)
        }
        int row_even = rb * 8 + 2 * c;
        *reinterpret_cast<uint4*>(lds + lds_off<BK>(row_even, kb)) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        *reinterpret_cast<uint4*>(lds + lds_off<BK>(row_even + 1, kb)) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
      }
    }
  }
};

__device__ __forceinline__ f32x4_t load_bf16x4_as_f32(const uint16_t* p) {
  uint2 raw = *reinterpret_cast<const uint2*>(p);
  f32x4_t v;
  v[0] = __uint_as_float(raw.x << 16);
  v[1] = __uint_as_float(raw.x & 0xffff0000u);
  v[2] = __uint_as_float(raw.y << 16);
  v[3] = __uint_as_float(raw.y & 0xffff0000u);
  return v;
}

__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Sum over the workgroup in a fixed order (same result in every workgroup and every run).
template <int NT>
__device__ __forceinline__ float block_sum_f32(float v, float* red) {
  v = wave_sum_f32(v);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = 0.0f;
#pragma unroll
  for (int w = 0; w < NT / 64; ++w) t += red[w];
  __syncthreads();
  return t;
}

// The diagonal shift s of this workgroup's matrix and the effective coefficients of product and addends
// (returned by value: scalars handed out by reference end up in scratch memory).
struct Scalars {
  float shift, alpha, beta, beta2;
};
template <int NT>
__device__ __forceinline__ Scalars resolve_shift(const GemmParams& p, int64_t batch, float* red, bool first_of_batch) {
  float s = 0.0f, alpha = p.alpha, beta = p.beta, beta2 = p.beta2;
  if (p.shift_mode == SHIFT_GRAM) {
    float part = 0.0f;
    const float* sl = p.slots_in + batch * p.nslots_in;
    for (int i = threadIdx.x; i < p.nslots_in; i += NT) part += sl[i];
    s = block_sum_f32<NT>(part, red) / (float)p.M;
    if (first_of_batch && threadIdx.x == 0) p.shift_io[batch] = s;
  } else if (p.shift_mode == SHIFT_POLY) {
    s = p.shift_io[batch];
    beta = beta + 2.0f * p.cc * s;  // B' = c A'^2 + (b + 2 c s) A'
  } else if (p.shift_mode == SHIFT_APPLY) {
    s = p.shift_io[batch];
    beta = beta + p.cb * s + p.cc * s * s;  // X' = (a + b s + c s^2) X + B' X
  } else if (p.shift_mode >= SHIFT_GROUP_POLY) {
    s = p.shift_io[batch];
    // walk the recursion up to this launch's step: sk = s_k, e = e_k, before = alpha_{k-1}
    float sk = s, before = 1.0f, e = 0.0f;
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      if (j > p.stage) break;
      e = p.co[j][0] + p.co[j][1] * sk + p.co[j][2] * sk * sk;
      if (j < p.stage) {
        before *= e;
        sk = e * e * sk;
      }
    }
    const int mode = p.shift_mode;
    // (selects instead of p.co[p.stage]: a dynamically indexed kernel argument would be copied to scratch)
    const float bk = p.stage == 0 ? p.co[0][1] : p.stage == 1 ? p.co[1][1] : p.co[2][1];
    const float ck = p.stage == 0 ? p.co[0][2] : p.stage == 1 ? p.co[1][2] : p.co[2][2];
    beta = mode == SHIFT_GROUP_POLY ? bk + 2.0f * ck * sk : mode == SHIFT_GROUP_APPLY ? before * e : e;
    beta2 = mode == SHIFT_GROUP_T ? sk : mode == SHIFT_GROUP_A ? e * sk : mode == SHIFT_GROUP_Q ? before : beta2;
  }
  if (p.xscale != nullptr) {
    const float r = p.xscale[batch];
    if (p.shift_mode == SHIFT_GRAM) {
      alpha *= r * r;
    } else {
      alpha *= r;
      beta *= r;
    }
  }
  return Scalars{s, alpha, beta, beta2};
}

// Epilogue shared by both kernels.  MI names the MFMA tile the accumulators come from:
//   MI = 32 (f32x16): a lane owns output row m = m_base + 32 i + (lane & 31) and, for each (j, g), the four
//                     columns n .. n+3 with n = n_base + 32 j + 8 g + 4 (lane >> 5)
//   MI = 16 (f32x4):  row m = m_base + 16 i + (lane & 15), columns n .. n+3 with n = n_base + 16 j + 4 (lane >> 4)
template <int MODE, bool OUT_F32, bool GUARD, int FM, int FN, int NT, int MI = 32, class ACC = f32x16_t>
__device__ __forceinline__ void tile_epilogue(const GemmParams& p, ACC (&acc)[FM][FN], int m_base, int n_base,
                                              int lane, int64_t batch, bool diag, float alpha, float beta, float shift,
                                              float* red, float beta2 = 0.0f) {
  constexpr int G = MI == 32 ? 4 : 1;
  const int frow = lane & (MI - 1), fk = lane / MI;
  const uint16_t* __restrict__ Cb = p.Cin ? p.Cin + batch * p.c_bs : nullptr;
  const bool use_c = beta != 0.0f && Cb != nullptr;
  const uint16_t* __restrict__ Cb2 = (MODE == MODE_SYRK && p.Cin2) ? p.Cin2 + batch * p.c_bs : nullptr;
  const bool use_c2 = beta2 != 0.0f && Cb2 != nullptr;
  // All Cin pieces are requested before the first store (stores may alias Cin as far as the compiler knows, so
  // loads left between them would each wait out a full memory latency).
  constexpr bool HOIST_C = FM * FN * G * 2 <= 96;  // register budget
  uint2 cpre[HOIST_C ? FM : 1][HOIST_C ? FN : 1][G];
  if (HOIST_C && use_c) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const int m = m_base + i * MI + frow, n = n_base + j * MI + (MI == 32 ? 8 * g : 0) + 4 * fk;
          cpre[i][j][g] = make_uint2(0u, 0u);
          if (!GUARD || (m < p.M && n < p.N)) cpre[i][j][g] = *reinterpret_cast<const uint2*>(Cb + (int64_t)m * p.ldc + n);
        }
  }
  float ssq = 0.0f;
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    const int m = m_base + i * MI + frow;
#pragma unroll
    for (int j = 0; j < FN; ++j) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const int n = n_base + j * MI + (MI == 32 ? 8 * g : 0) + 4 * fk;
        if (GUARD && (m >= p.M || n >= p.N)) continue;
        f32x4_t v;
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = alpha * acc[i][j][4 * g + r];
        if (use_c) {
          f32x4_t c;
          if (HOIST_C) {
            const uint2 raw = cpre[i][j][g];
            c[0] = __uint_as_float(raw.x << 16);
            c[1] = __uint_as_float(raw.x & 0xffff0000u);
            c[2] = __uint_as_float(raw.y << 16);
            c[3] = __uint_as_float(raw.y & 0xffff0000u);
          } else {
            c = load_bf16x4_as_f32(Cb + (int64_t)m * p.ldc + n);
          }
#pragma unroll
          for (int r = 0; r < 4; ++r) v[r] = __builtin_fmaf(beta, c[r], v[r]);
        }
        if (use_c2) {
          const f32x4_t c = load_bf16x4_as_f32(Cb2 + (int64_t)m * p.ldc + n);
#pragma unroll
          for (int r = 0; r < 4; ++r) v[r] = __builtin_fmaf(beta2, c[r], v[r]);
        }
        if (MODE == MODE_SYRK && p.shift_mode == SHIFT_GRAM && diag) {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (n + r == m) v[r] -= shift;
        }
        if (MODE == MODE_GEMM) {
#pragma unroll
          for (int r = 0; r < 4; ++r) ssq = __builtin_fmaf(v[r], v[r], ssq);
        }
        if (OUT_F32) {
          float* o = reinterpret_cast<float*>(p.Out) + batch * p.o_bs + (int64_t)m * p.ldo + n;
          f32x4_t w;
#pragma unroll
          for (int r = 0; r < 4; ++r) w[r] = v[r] * p.out_scale;
          if (p.out_accum != 0.0f) {
            const f32x4_t old = *reinterpret_cast<const f32x4_t*>(o);
#pragma unroll
            for (int r = 0; r < 4; ++r) w[r] = __builtin_fmaf(p.out_accum, old[r], w[r]);
          }
          *reinterpret_cast<f32x4_t*>(o) = w;
        } else {
          uint16_t* ob = reinterpret_cast<uint16_t*>(p.Out) + batch * p.o_bs;
          bf16x4_t h = __builtin_convertvector(v, bf16x4_t);
          if (MODE == MODE_GEMM) {
            *reinterpret_cast<bf16x4_t*>(ob + (int64_t)m * p.ldo + n) = h;
          } else {
            const uint2 hb = __builtin_bit_cast(uint2, h);
            const uint16_t ev[4] = {(uint16_t)(hb.x & 0xffffu), (uint16_t)(hb.x >> 16), (uint16_t)(hb.y & 0xffffu),
                                    (uint16_t)(hb.y >> 16)};
            if (!diag) {
              *reinterpret_cast<uint2*>(ob + (int64_t)m * p.ldo + n) = hb;
              if (!p.skip_upper) {
#pragma unroll
                for (int r = 0; r < 4; ++r) ob[(int64_t)(n + r) * p.ldo + m] = ev[r];
              }
            } else if (p.skip_upper) {
              *reinterpret_cast<uint2*>(ob + (int64_t)m * p.ldo + n) = hb;
            } else {
              // Diagonal tile: the lower half is stored and mirrored, the computed upper half is
              // dropped, so the result is symmetric bit for bit by construction.
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                if (n + r <= m) ob[(int64_t)m * p.ldo + n + r] = ev[r];
                if (n + r < m) ob[(int64_t)(n + r) * p.ldo + m] = ev[r];
              }
            }
          }
        }
      }
    }
  }
  if (MODE == MODE_GEMM && p.slots_out != nullptr) {
    const float total = block_sum_f32<NT>(ssq, red);
    if (threadIdx.x == 0) p.slots_out[batch * p.slot_stride + p.slot_base + blockIdx.x] = total;
  }
}

// ---------------------------------------------------------------------------------------------
// The kernel.  grid = (tiles, batch); block = WGM*WGN wavefronts; dynamic LDS = 2 stages.
// ---------------------------------------------------------------------------------------------
template <int BM, int BN, int BK, int WGM, int WGN, bool P_KS, bool Q_KS, int MODE, bool OUT_F32>
__global__ void __launch_bounds__(WGM* WGN * 64) gemm_bf16_kernel(GemmParams p) {
  constexpr int NT = WGM * WGN * 64;
  constexpr int TM = BM / WGM, TN = BN / WGN;
  constexpr int FM = TM / 32, FN = TN / 32;
  constexpr int P_BYTES = BM * BK * 2, Q_BYTES = BN * BK * 2, STAGE = P_BYTES + Q_BYTES;
  static_assert(TM % 32 == 0 && TN % 32 == 0 && BK % 16 == 0, "tile shape");
  static_assert(MODE != MODE_SYRK || BM == BN, "SYRK needs square tiles");

  extern __shared__ __align__(16) char smem[];
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
  const uint16_t* __restrict__ Pb = p.P + batch * p.p_bs;
  const uint16_t* __restrict__ Qb = p.Q + batch * p.q_bs;

  TileLoader<BM, BK, NT, P_KS> lp;
  TileLoader<BN, BK, NT, Q_KS> lq;

  f32x16_t acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  const int nk = (p.K + BK - 1) / BK;
  lp.load(Pb, p.ldp, m0, 0, p.M, p.K, tid);
  lq.load(Qb, p.ldq, n0, 0, p.N, p.K, tid);
  lp.store(smem, tid);
  lq.store(smem + P_BYTES, tid);
  __syncthreads();

  const int frow = lane & 31, fk = lane >> 5;
  for (int kt = 0; kt < nk; ++kt) {
    const char* cur = smem + (kt & 1) * STAGE;
    char* nxt = smem + ((kt + 1) & 1) * STAGE;
    const bool more = (kt + 1) < nk;
    if (more) {
      lp.load(Pb, p.ldp, m0, (kt + 1) * BK, p.M, p.K, tid);
      lq.load(Qb, p.ldq, n0, (kt + 1) * BK, p.N, p.K, tid);
    }
#pragma unroll
    for (int q = 0; q < BK / 16; ++q) {
      bf16x8_t fp[FM], fq[FN];
#pragma unroll
      for (int i = 0; i < FM; ++i)
        fp[i] = *reinterpret_cast<const bf16x8_t*>(cur + lds_off<BK>(wm * TM + i * 32 + frow, 2 * q + fk));
#pragma unroll
      for (int j = 0; j < FN; ++j)
        fq[j] = *reinterpret_cast<const bf16x8_t*>(cur + P_BYTES + lds_off<BK>(wn * TN + j * 32 + frow, 2 * q + fk));
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fq[j], fp[i], acc[i][j], 0, 0, 0);
    }
    if (more) {
      lp.store(nxt, tid);
      lq.store(nxt + P_BYTES, tid);
    }
    __syncthreads();
  }

  const Scalars sc = resolve_shift<NT>(p, batch, red, blockIdx.x == 0);
  const bool diag = (MODE == MODE_SYRK) && (tm == tn);
  tile_epilogue<MODE, OUT_F32, true, FM, FN, NT>(p, acc, m0 + wm * TM, n0 + wn * TN, lane, batch, diag, sc.alpha, sc.beta,
                                                 sc.shift, red, sc.beta2);
}

}  // namespace mi
