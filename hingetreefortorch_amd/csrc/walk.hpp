// Device-side path walk shared by every kernel.
//
// Semantics pinned by the reference's HingeTreeCommon.h:157-178 (tree) and :72-91 (fern):
//   * the root margin seeds the running minimum and the update is a strict '<' on |margin|, so the first minimum on
//     the path wins;
//   * margin > 0 goes right, margin == 0 and NaN go left;
//   * bit i of the leaf key is the decision at level i (root = bit 0); this is not the heap order of the leaves;
//   * the selected vertex is a heap index for trees and a level for ferns.
// The translation units are compiled with -ffp-contract=off: margin = x - thr is a single rounded subtract.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ht {

template <typename Real>
struct WalkResult {
  uint32_t key;     // leaf key
  uint32_t vertex;  // index into thr/ord of the min-|margin| decision
  Real margin;      // its signed margin
};

__device__ __forceinline__ float ht_abs(float v) { return __builtin_fabsf(v); }
__device__ __forceinline__ double ht_abs(double v) { return __builtin_fabs(v); }

// Ordinals are validated by the caller; this only guarantees that a value which slipped through can never turn into
// an out-of-bounds address.
__device__ __forceinline__ int clamp_ordinal(int64_t o, int n) {
  const unsigned u = (unsigned)o;
  return int(u < (unsigned)n ? u : (unsigned)(n - 1));
}

template <typename Real>
__device__ __forceinline__ Real ht_sign(Real m) {
  return Real((Real(0) < m) - (m < Real(0)));
}

// `node(i)` returns (threshold, ordinal) of decision i; `feature(f)` returns this sample's value of feature f.
template <typename Real, bool FERN, typename NodeFn, typename FeatureFn>
__device__ __forceinline__ WalkResult<Real> walk(int depth, NodeFn node, FeatureFn feature) {
  WalkResult<Real> r;
  uint32_t v = 0;
  r.key = 0;
  r.vertex = 0;
  {
    Real th;
    int o;
    node(0u, th, o);
    r.margin = feature(o) - th;
  }
  Real best_abs = ht_abs(r.margin);
  for (int lvl = 0; lvl < depth; ++lvl) {
    const uint32_t at = FERN ? uint32_t(lvl) : v;
    Real th;
    int o;
    node(at, th, o);
    const Real m = feature(o) - th;
    const uint32_t bit = (m > Real(0)) ? 1u : 0u;
    const Real a = ht_abs(m);
    if (a < best_abs) {
      best_abs = a;
      r.margin = m;
      r.vertex = at;
    }
    r.key |= bit << lvl;
    v = 2u * v + 1u + bit;
  }
  return r;
}

}  // namespace ht
