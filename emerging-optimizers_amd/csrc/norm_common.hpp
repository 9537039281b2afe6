// Pieces of the Frobenius normalisation that more than one translation unit uses: the momentum source of the fused
// optimizer step and the streaming load of the float32 input.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm_engine.hpp"

namespace mi {

// Frobenius norms in this range let the divide be deferred to the consumers of X: squares of the entries neither
// overflow nor vanish in float32.
static constexpr float NORM_DEFER_MIN = 1e-10f, NORM_DEFER_MAX = 1e10f;

// Momentum source of the fused optimizer step (orthogonalized_optimizer.py:185-192 of the reference):
//   buf <- buf + (1 - beta) (g - buf)           [buf.lerp_(grad, 1 - beta)]
//   d    = nesterov ? buf - (buf - g) (1 - beta) [grad.lerp(buf, beta)] : buf
// lerp follows torch's two-branch formula (weight < 0.5: start + w (end - start); else end - (end - start)(1 - w)).
struct MomentumSrc {
  float* buf;     // momentum buffer, updated in place by the sum-of-squares pass; null: plain input
  float beta;
  int nesterov;
};
__device__ __forceinline__ float torch_lerp(float start, float end, float w) {
  const float diff = end - start;
  return w < 0.5f ? start + w * diff : end - diff * (1.0f - w);
}
__device__ __forceinline__ float momentum_direction(float g, float buf_new, float beta, int nesterov) {
  return nesterov ? torch_lerp(g, buf_new, beta) : buf_new;
}

// The float32 input is read exactly once on this path: a non-temporal load keeps it from displacing the bf16 copy
// (which the first Gram product reads next) from the caches.  Measured at 4096 x 14336: 65 -> 60 us for this pass and
// 200 -> 193 us for the Gram product that follows; a non-temporal store of the bf16 copy costs 7 us instead.
__device__ __forceinline__ f32x4_t stream_load4(const float* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const f32x4_t*>(p));
}

}  // namespace mi
