// 128-row matrices (one attention head each): the product X' = beta X + alpha S X that ends a group of Newton-Schulz
// steps, together with the split-K partial Gram matrices of X' that the next group starts from.
//
// The general GEMM+AXPY kernel runs this shape (K = 128: two K tiles) as 512 independent tiles that each pay a
// prologue and an epilogue, reads X twice (as operand and as addend), and the next group's Gram kernel reads X' a
// third time.  Here one workgroup owns 512 consecutive columns of one head -- the same slice that a Gram partial
// covers -- and walks them in slabs of 128 columns that it keeps in LDS: a slab is read from memory once, serves as the
// K-strided operand of S X (transpose reads), as the addend, then holds X' in place, from where it is written out with
// whole rows and multiplied by itself for the partial Gram matrix.  S stays in registers as MFMA fragments.  The next
// slab is on its way from memory into registers while the current one is worked on.
#include "launch_impl.hpp"

namespace mi {

static constexpr int HA_M = 128;       // rows of a matrix = K of the product
static constexpr int HA_W = 128;       // columns of a slab
static constexpr int HA_SPLIT = 512;   // columns of a workgroup = K range of one Gram partial
static constexpr int HA_NT = 512;      // 8 wavefronts, two per SIMD: one's LDS and MFMA latencies hide behind the other's work
static constexpr int HA_ROWB = HA_W * 2, HA_CH = HA_W / 8;  // bytes and 16-byte chunks of a slab row
static constexpr int HA_SLAB_BYTES = HA_M * HA_ROWB;        // 32 KB
static constexpr int HA_PRE = HA_SLAB_BYTES / 16 / HA_NT;   // 16-byte chunks of a slab per thread
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));  // 16 bytes in flight between memory and LDS

// Byte offset of chunk c8 (8 columns) of slab row k: the layout of a K-strided operand tile (gemm_fast.hpp), rows
// rotated by ks_rot so that transpose reads and row reads both spread over the banks.
__device__ __forceinline__ int ha_chunk(int k, int c8) { return k * HA_ROWB + (((c8 + ks_rot(k)) & (HA_CH - 1)) << 4); }

template <bool OUT_F32>
__global__ void __launch_bounds__(HA_NT) head_apply_kernel(GemmParams p, float* gram_next, int splits) {
  // two slabs of X (the one worked on, the next one) and, for the bf16 result, two slabs of X'
  __shared__ __align__(1024) char slab_in[2][HA_SLAB_BYTES];
  __shared__ __align__(1024) char slab_out[OUT_F32 ? 1 : 2][OUT_F32 ? 16 : HA_SLAB_BYTES];
  __shared__ float red[HA_NT / 64];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t b = blockIdx.x / splits;
  const int s = blockIdx.x % splits;
  const int64_t c_begin = (int64_t)s * HA_SPLIT;

  const uint16_t* __restrict__ X = p.Q + b * p.q_bs;
  const uint16_t* __restrict__ Sm = p.P + b * p.p_bs;

  // S as fragments of the P operand: rows 16 wave + lane % 16, k = 32 q + 8 (lane / 16) .. + 7
  bf16x8_t sfrag[4];
#pragma unroll
  for (int q = 0; q < 4; ++q)
    sfrag[q] = *reinterpret_cast<const bf16x8_t*>(Sm + (int64_t)(16 * wave + (lane & 15)) * p.ldp + 32 * q + 8 * (lane >> 4));

  // slab <-> threads: chunk id tid + 512 u covers row (tid >> 4) + 32 u, chunk tid & 15
  const int ck = tid >> 4, cc = tid & 15;
  u32x4_t pre[HA_PRE];
  auto fetch_slab = [&](int t) {
#pragma unroll
    for (int u = 0; u < HA_PRE; ++u)
      pre[u] = *reinterpret_cast<const u32x4_t*>(X + (int64_t)(ck + 32 * u) * p.ldq + c_begin + t * HA_W + 8 * cc);
  };
  auto park_slab = [&](char* buf) {
#pragma unroll
    for (int u = 0; u < HA_PRE; ++u) *reinterpret_cast<u32x4_t*>(buf + ha_chunk(ck + 32 * u, cc)) = pre[u];
  };
  uint32_t ks_s, ks_r;  // lane constants of the transpose reads (columns of the slab = rows of the Q operand)
  ks16_consts<HA_W>(lane, 0, ks_s, ks_r);

  // partial Gram matrix of X': wavefront w owns rows 16 w .. + 15 and the columns up to its diagonal block (the
  // part above the diagonal is never read)
  const bool want_gram = !OUT_F32 && gram_next != nullptr;
  f32x4_t gacc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) gacc[j] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

  float ssq = 0.0f;
  fetch_slab(0);
  // (the scalars are resolved while the first loads are on their way)
  const Scalars sc = resolve_shift<HA_NT>(p, b, red, s == 0);
  const float alpha = sc.alpha, beta = sc.beta;
  const bool use_c = beta != 0.0f && p.Cin != nullptr;  // (the addend is X itself: p.Cin == p.Q)
  park_slab(slab_in[0]);
  __syncthreads();
  constexpr int SLABS = HA_SPLIT / HA_W;
  // (unrolled: with a run-time slab index the prefetch registers, written under a condition, ended up in scratch memory)
  static_for<SLABS>([&](auto tc) {
    constexpr int t = decltype(tc)::value;
    char* cur = slab_in[t & 1];
    char* res = slab_out[OUT_F32 ? 0 : (t & 1)];
    if constexpr (t + 1 < SLABS) fetch_slab(t + 1);  // in flight during everything below
    // ---- S X on the slab: rows 16 wave .. + 15, all 128 columns ----
    f32x4_t acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    const uint32_t cur_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)cur;
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int j = 0; j < 8; ++j)
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fast_frag16_ks<HA_W>(cur_lds, ks_s, ks_r, j, q), sfrag[q], acc[j], 0, 0, 0);
    // The next slab of X goes into the buffer whose readers (fragments and addends of the previous pass) finished
    // before the barrier of the previous pass.  With float32 output this happens before the epilogue: the wait for
    // the loads would otherwise also wait for the stores of the epilogue, which share their counter.
    if constexpr (OUT_F32 && t + 1 < SLABS) park_slab(slab_in[(t + 1) & 1]);
    // ---- epilogue: a lane owns row m = 16 wave + lane % 16, columns n .. n + 3 with n = 16 j + 4 (lane / 16) ----
    const int m = 16 * wave + (lane & 15);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int n = 16 * j + 4 * (lane >> 4);
      const int at = ha_chunk(m, n >> 3) + (n & 7) * 2;
      f32x4_t v;
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] = alpha * acc[j][r];
      if (use_c) {
        const uint2 raw = *reinterpret_cast<const uint2*>(cur + at);
        v[0] = __builtin_fmaf(beta, __uint_as_float(raw.x << 16), v[0]);
        v[1] = __builtin_fmaf(beta, __uint_as_float(raw.x & 0xffff0000u), v[1]);
        v[2] = __builtin_fmaf(beta, __uint_as_float(raw.y << 16), v[2]);
        v[3] = __builtin_fmaf(beta, __uint_as_float(raw.y & 0xffff0000u), v[3]);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) ssq = __builtin_fmaf(v[r], v[r], ssq);
      if constexpr (OUT_F32) {
        float* o = reinterpret_cast<float*>(p.Out) + b * p.o_bs + (int64_t)m * p.ldo + c_begin + t * HA_W + n;
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
        *reinterpret_cast<uint2*>(res + at) = __builtin_bit_cast(uint2, __builtin_convertvector(v, bf16x4_t));  // same layout as the slab of X
      }
    }
    if constexpr (!OUT_F32 && t + 1 < SLABS) park_slab(slab_in[(t + 1) & 1]);
    if constexpr (t + 1 < SLABS || !OUT_F32) __syncthreads();  // X' of this pass and X of the next one are complete
    if constexpr (!OUT_F32) {
      // (the buffer of X' is written again two passes on, behind the barrier of the next pass)
      uint16_t* __restrict__ ob = reinterpret_cast<uint16_t*>(p.Out) + b * p.o_bs + c_begin + t * HA_W;
#pragma unroll
      for (int u = 0; u < HA_PRE; ++u)
        *reinterpret_cast<u32x4_t*>(ob + (int64_t)(ck + 32 * u) * p.ldo + 8 * cc) = *reinterpret_cast<const u32x4_t*>(res + ha_chunk(ck + 32 * u, cc));
      if (want_gram) {
        // G += X' X'^T over the 128 columns of the slab (4 k-steps); both operands are rows of the slab
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const bf16x8_t fp = *reinterpret_cast<const bf16x8_t*>(res + ha_chunk(16 * wave + (lane & 15), 4 * q + (lane >> 4)));
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            if (j > wave) continue;  // (uniform)
            const bf16x8_t fq = *reinterpret_cast<const bf16x8_t*>(res + ha_chunk(16 * j + (lane & 15), 4 * q + (lane >> 4)));
            gacc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fq, fp, gacc[j], 0, 0, 0);
          }
        }
      }
    }
  });
  // ---- what the workgroup leaves: its partial sum of squares and its partial Gram matrix ----
  const float total = block_sum_f32<HA_NT>(ssq, red);
  if (p.slots_out != nullptr && tid == 0) p.slots_out[b * p.slot_stride + p.slot_base + s] = total;
  if (want_gram) {
    float* __restrict__ g = gram_next + (b * splits + s) * (int64_t)(HA_M * HA_M);
    const int m = 16 * wave + (lane & 15);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (j > wave) continue;
      *reinterpret_cast<f32x4_t*>(g + (int64_t)m * HA_M + 16 * j + 4 * (lane >> 4)) = gacc[j];
    }
  }
}

bool head_apply_supported(const GemmParams& p, int64_t batch, int splits) {
  return p.M == HA_M && p.K == HA_M && p.N > 0 && p.N % HA_SPLIT == 0 && splits == p.N / HA_SPLIT && batch > 0 &&
         batch * splits <= (int64_t)1 << 30 && p.ldp >= HA_M && p.ldq >= p.N && p.ldo >= p.N && p.ldp % 8 == 0 && p.ldq % 8 == 0 &&
         p.ldo % 8 == 0 && p.q_bs % 8 == 0 && p.p_bs % 8 == 0 && p.o_bs % 8 == 0 && (p.Cin == nullptr || p.Cin == p.Q) && p.Cin2 == nullptr;
}

int launch_head_apply(const GemmParams& p, int64_t batch, int splits, float* gram_next, bool out_f32, hipStream_t stream) {
  if (!head_apply_supported(p, batch, splits))
    return fail(MI_ERR_UNSUPPORTED_SHAPE, "internal: per-head product on %d x %d (K = %d), %d slices", p.M, p.N, p.K, splits);
  if (out_f32 && gram_next != nullptr) return fail(MI_ERR_BAD_ARG, "internal: the Gram partials need the bf16 result");
  if (p.out_transposed) return fail(MI_ERR_UNSUPPORTED_SHAPE, "internal: the slab kernel has no transposed output");
  GemmParams q = p;
  if (q.slot_stride == 0) q.slot_stride = splits;
  if (int rc = check_slots(q, splits)) return rc;
  dim3 grid((unsigned)(batch * splits)), block(HA_NT);
  MI_OTHER_LAUNCH();
  MI_FOOTPRINT("multiplier S", q.P, 2, batch, q.p_bs, HA_M, q.ldp, HA_M);
  MI_FOOTPRINT("X", q.Q, 2, batch, q.q_bs, HA_M, q.ldq, q.N);
  MI_FOOTPRINT("X'", q.Out, out_f32 ? 4 : 2, batch, q.o_bs, HA_M, q.ldo, q.N);
  MI_FOOTPRINT("Gram partials of X'", gram_next, 4, batch, (int64_t)splits * HA_M * HA_M, splits, HA_M * HA_M, HA_M * HA_M);
#ifdef MI_HOST_CHECK
  host_check::scalar_footprints(q, batch, splits);
#endif
  if (out_f32)
    hipLaunchKernelGGL(head_apply_kernel<true>, grid, block, 0, stream, q, gram_next, splits);
  else
    hipLaunchKernelGGL(head_apply_kernel<false>, grid, block, 0, stream, q, gram_next, splits);
  g_last_launch = LastLaunch{splits, HA_M, HA_SPLIT, 3};
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
  return MI_OK;
}

// ---------------------------------------------------------------------------------------------
// The pass over the float32 input of 128-row matrices that starts a call: sum of squares, bf16 cast (unnormalised: the
// divide by the norm is left to the consumers) and, because the slab that was just cast sits in LDS anyway, the
// split-K partial Gram matrices of the cast -- the first group of steps then needs no Gram kernel that reads X again.
// One workgroup per (matrix, slice of 512 columns), slabs of 128 columns as above.
//
// FINALIZE = false is that pass.  FINALIZE = true follows it: every workgroup adds the partial sums of its matrix, and
// for a norm in the range where the divide may be deferred that is all (one thread per matrix leaves norm, scale and
// the squared norm of the normalised matrix); for a norm outside it the workgroup does the work again on x / norm:
// the cast and the partial Gram matrices are replaced by those of the normalised matrix, and the scale is 1.
// ---------------------------------------------------------------------------------------------
struct HeadFrontArgs {
  const float* x;     // [batch][128][n] float32 (the gradient, with a momentum source)
  int64_t n;
  int splits;         // n / 512
  float eps;
  MomentumSrc mom;
  uint16_t* xb;       // [batch][128][n] bf16
  double* partials;   // [batch][splits]
  float* gram;        // [batch][splits][128][128]
  float* norm;        // [batch] or null
  float* sumsq_out;   // [batch] or null
  float* xscale;      // [batch]
};

template <bool FINALIZE>
__global__ void __launch_bounds__(HA_NT) head_front_kernel(HeadFrontArgs a) {
  __shared__ __align__(1024) char slab[2][HA_SLAB_BYTES];
  __shared__ double red_d[HA_NT / 64];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t b = blockIdx.x / a.splits;
  const int s = blockIdx.x % a.splits;
  float divisor = 1.0f;
  if constexpr (FINALIZE) {
    double tot = 0.0;
    for (int i = 0; i < a.splits; ++i) tot += a.partials[b * a.splits + i];  // (same order in every thread and workgroup)
    divisor = fmaxf(sqrtf((float)tot), a.eps);
    const bool deferred = divisor >= NORM_DEFER_MIN && divisor <= NORM_DEFER_MAX;  // false for NaN
    if (s == 0 && tid == 0) {
      if (a.norm) a.norm[b] = divisor;
      a.xscale[b] = deferred ? 1.0f / divisor : 1.0f;
      if (a.sumsq_out) {
        // squared Frobenius norm of the normalised matrix: 1 unless the divisor was clamped
        const float ratio = sqrtf((float)tot) / divisor;
        a.sumsq_out[b] = (divisor > 0.0f && ratio == ratio) ? ratio * ratio : 0.0f;
      }
    }
    if (deferred) return;
  }

  // slab <-> threads as in head_apply_kernel: 8 columns of row (tid >> 4) + 32 u, chunk tid & 15
  const int ck = tid >> 4, cc = tid & 15;
  const int64_t base = b * (int64_t)HA_M * a.n + (int64_t)s * HA_SPLIT + 8 * cc;
  const float* __restrict__ xs = a.x + base;
  float* __restrict__ ms = a.mom.buf ? a.mom.buf + base : nullptr;
  uint16_t* __restrict__ os = a.xb + base;
  const float keep = 1.0f - a.mom.beta;
  f32x4_t pre[HA_PRE][2], mpre[HA_PRE][2];
  auto fetch = [&](int t) {
#pragma unroll
    for (int u = 0; u < HA_PRE; ++u) {
      const int64_t at = (int64_t)(ck + 32 * u) * a.n + t * HA_W;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        pre[u][h] = FINALIZE ? *reinterpret_cast<const f32x4_t*>(xs + at + 4 * h) : stream_load4(xs + at + 4 * h);
        if (ms) mpre[u][h] = *reinterpret_cast<const f32x4_t*>(ms + at + 4 * h);
      }
    }
  };
  f32x4_t gacc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) gacc[j] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
  f32x4_t ssq = {0.0f, 0.0f, 0.0f, 0.0f};
  constexpr int SLABS = HA_SPLIT / HA_W;
  fetch(0);
  static_for<SLABS>([&](auto tc) {
    constexpr int t = decltype(tc)::value;
    char* cur = slab[t & 1];
#pragma unroll
    for (int u = 0; u < HA_PRE; ++u) {
      const int64_t at = (int64_t)(ck + 32 * u) * a.n + t * HA_W;
      uint2 half[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        f32x4_t v = pre[u][h];
        if (ms) {
          f32x4_t m = mpre[u][h];
          if constexpr (!FINALIZE) {  // (the second pass finds the buffer updated)
#pragma unroll
            for (int e = 0; e < 4; ++e) m[e] = torch_lerp(m[e], v[e], keep);
            *reinterpret_cast<f32x4_t*>(ms + at + 4 * h) = m;
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = momentum_direction(v[e], m[e], a.mom.beta, a.mom.nesterov);
        }
        if constexpr (FINALIZE) {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = v[e] / divisor;
        } else {
          // squares are formed in float32: tiny inputs underflow exactly like a float32 reduction
#pragma unroll
          for (int e = 0; e < 4; ++e) ssq[e] = __builtin_fmaf(v[e], v[e], ssq[e]);
        }
        half[h] = __builtin_bit_cast(uint2, __builtin_convertvector(v, bf16x4_t));
      }
      const u32x4_t chunk = {half[0].x, half[0].y, half[1].x, half[1].y};
      *reinterpret_cast<u32x4_t*>(os + at) = chunk;
      *reinterpret_cast<u32x4_t*>(cur + ha_chunk(ck + 32 * u, cc)) = chunk;
    }
    if constexpr (t + 1 < SLABS) fetch(t + 1);  // in flight during the products below
    // One barrier per slab: the buffer written above was last read by the products of two slabs ago, which every
    // wavefront finished before it arrived at the barrier of the previous slab.
    __syncthreads();
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const bf16x8_t fp = *reinterpret_cast<const bf16x8_t*>(cur + ha_chunk(16 * wave + (lane & 15), 4 * q + (lane >> 4)));
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (j > wave) continue;  // (uniform)
        const bf16x8_t fq = *reinterpret_cast<const bf16x8_t*>(cur + ha_chunk(16 * j + (lane & 15), 4 * q + (lane >> 4)));
        gacc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fq, fp, gacc[j], 0, 0, 0);
      }
    }
  });
  if constexpr (!FINALIZE) {
    // the cross-thread tree is carried in float64, so the result does not depend on its shape
    double v = (double)((ssq[0] + ssq[1]) + (ssq[2] + ssq[3]));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
    if (lane == 0) red_d[wave] = v;
    __syncthreads();
    if (tid == 0) {
      double tot = 0.0;
      for (int w = 0; w < HA_NT / 64; ++w) tot += red_d[w];
      a.partials[b * a.splits + s] = tot;
    }
  }
  float* __restrict__ g = a.gram + (b * a.splits + s) * (int64_t)(HA_M * HA_M);
  const int m = 16 * wave + (lane & 15);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    if (j > wave) continue;
    *reinterpret_cast<f32x4_t*>(g + (int64_t)m * HA_M + 16 * j + 4 * (lane >> 4)) = gacc[j];
  }
}

static inline bool ha_aligned16(const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; }

bool head_front_supported(const float* x, int64_t batch, int64_t n, const MomentumSrc& mom) {
  return x != nullptr && batch > 0 && n > 0 && n % HA_SPLIT == 0 && batch * (n / HA_SPLIT) <= (int64_t)1 << 30 && ha_aligned16(x) &&
         ha_aligned16(mom.buf);
}

int launch_head_front(const float* x, int64_t batch, int64_t n, float eps, MomentumSrc mom, uint16_t* xb, double* partials,
                      float* gram, float* norm, float* sumsq_out, float* xscale, hipStream_t stream) {
  if (!head_front_supported(x, batch, n, mom) || !xb || !partials || !gram || !xscale || !ha_aligned16(xb) || !ha_aligned16(gram))
    return fail(MI_ERR_UNSUPPORTED_SHAPE, "internal: per-head input pass on %lld matrices of 128 x %lld", (long long)batch, (long long)n);
  HeadFrontArgs a{x, n, (int)(n / HA_SPLIT), eps, mom, xb, partials, gram, norm, sumsq_out, xscale};
  dim3 grid((unsigned)(batch * a.splits)), block(HA_NT);
  MI_OTHER_LAUNCH();
  MI_FOOTPRINT("input", x, 4, batch, HA_M * n, HA_M, n, n);
  MI_FOOTPRINT("momentum buffer", mom.buf, 4, batch, HA_M * n, HA_M, n, n);
  MI_FOOTPRINT("bf16 copy", xb, 2, batch, HA_M * n, HA_M, n, n);
  MI_FOOTPRINT("partial sums of squares", partials, 8, batch, a.splits, 1, a.splits, a.splits);
  MI_FOOTPRINT("Gram partials", gram, 4, batch, (int64_t)a.splits * HA_M * HA_M, a.splits, HA_M * HA_M, HA_M * HA_M);
  MI_FOOTPRINT("norm", norm, 4, 1, 0, 1, batch, batch);
  MI_FOOTPRINT("squared norm of the result", sumsq_out, 4, 1, 0, 1, batch, batch);
  MI_FOOTPRINT("input scale", xscale, 4, 1, 0, 1, batch, batch);
  hipLaunchKernelGGL(head_front_kernel<false>, grid, block, 0, stream, a);
  hipLaunchKernelGGL(head_front_kernel<true>, grid, block, 0, stream, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MI_ERR_LAUNCH, "kernel launch failed: %s", hipGetErrorString(e));
  return MI_OK;
}

}  // namespace mi
