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
  uint32_t ord;     // the feature that decision tests
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

// A decision vertex as the kernels read it: threshold and (range-clamped) ordinal in one naturally aligned load.
template <typename Real>
struct Node;
template <>
struct __align__(8) Node<float> {
  float thr;
  int ord;
};
template <>
struct __align__(16) Node<double> {
  double thr;
  long long ord;
};

// N independent walks advanced level by level in one loop, so that their dependent load chains overlap.
// `node(i, at)` returns the packed vertex `at` (heap index, or level for a fern) of walk i, `feature(i, f)` returns
// walk i's sample value of feature f.
template <typename Real, bool FERN, int N, typename NodeFn, typename FeatureFn>
__device__ __forceinline__ void walk_many_fn(int depth, NodeFn node, FeatureFn feature, WalkResult<Real> (&r)[N]) {
  uint32_t v[N];
  Real best_abs[N];
#pragma unroll
  for (int i = 0; i < N; ++i) {
    v[i] = 0;
    r[i].key = 0;
    r[i].vertex = 0;
    r[i].ord = 0;
    r[i].margin = Real(0);
    best_abs[i] = Real(0);
  }
  for (int lvl = 0; lvl < depth; ++lvl) {
    Node<Real> n[N];
#pragma unroll
    for (int i = 0; i < N; ++i) n[i] = node(i, FERN ? uint32_t(lvl) : v[i]);
    Real m[N];
#pragma unroll
    for (int i = 0; i < N; ++i) m[i] = feature(i, int(n[i].ord)) - n[i].thr;
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const uint32_t at = FERN ? uint32_t(lvl) : v[i];
      const uint32_t bit = (m[i] > Real(0)) ? 1u : 0u;
      const Real a = ht_abs(m[i]);
      // level 0 seeds the minimum unconditionally (also when the root margin is NaN, which then sticks)
      if (lvl == 0 || a < best_abs[i]) {
        best_abs[i] = a;
        r[i].margin = m[i];
        r[i].vertex = at;
        r[i].ord = uint32_t(n[i].ord);
      }
      r[i].key |= bit << lvl;
      v[i] = 2u * v[i] + 1u + bit;
    }
  }
}

// The same with the vertices of walk i in the array nodes[i].
template <typename Real, bool FERN, int N, typename FeatureFn>
__device__ __forceinline__ void walk_many(int depth, const Node<Real> *const (&nodes)[N], FeatureFn feature,
                                          WalkResult<Real> (&r)[N]) {
  walk_many_fn<Real, FERN, N>(depth, [&](int i, uint32_t at) { return nodes[i][at]; }, feature, r);
}

// Leaner form of walk_many_fn for walks whose vertices and features both sit in LDS (little latency to hide, so the
// instruction count is what matters). The decisions are collected most significant bit first in `path` -- which is
// also the index of the current vertex inside its level, so the heap index needs no separate update -- and the leaf
// key (decision of level i in bit i) is the bit reversal of the finished path. TRACK = false skips the selected
// vertex / ordinal / signed margin (forward pass): r.margin then holds |margin|. TRACK = true carries the signed
// margin of the selected vertex as the running minimum (compared by magnitude) and beside it ONE word, level << 26 |
// ordinal (ordinals below 2^26, depth at most 32), from which the selected vertex is rebuilt once the path is
// complete: two selects per level instead of four.
constexpr int kPathLevelShift = 26;
template <typename Real, bool FERN, bool TRACK, int N, typename NodeFn, typename FeatureFn>
__device__ __forceinline__ void walk_paths(int depth, NodeFn node, FeatureFn feature, WalkResult<Real> (&r)[N]) {
  uint32_t path[N], info[N];
  Real best[N];  // TRACK: signed margin of the selected vertex; else its magnitude
#pragma unroll
  for (int i = 0; i < N; ++i) {
    path[i] = 0;
    info[i] = 0;
    best[i] = Real(0);
  }
  for (int lvl = 0; lvl < depth; ++lvl) {
    const uint32_t first = FERN ? uint32_t(lvl) : (1u << lvl) - 1u;  // wave uniform
    const uint32_t lvl_tag = uint32_t(lvl) << kPathLevelShift;        // wave uniform
    Node<Real> n[N];
#pragma unroll
    for (int i = 0; i < N; ++i) n[i] = node(i, FERN ? first : first + path[i]);
    Real m[N];
#pragma unroll
    for (int i = 0; i < N; ++i) m[i] = feature(i, int(n[i].ord)) - n[i].thr;
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if (TRACK) {
        if (lvl == 0 || ht_abs(m[i]) < ht_abs(best[i])) {
          best[i] = m[i];
          info[i] = lvl_tag | uint32_t(n[i].ord);
        }
      } else {
        const Real a = ht_abs(m[i]);
        if (lvl == 0 || a < best[i]) best[i] = a;
      }
      path[i] = path[i] + path[i] + ((m[i] > Real(0)) ? 1u : 0u);
    }
  }
#pragma unroll
  for (int i = 0; i < N; ++i) {
    r[i].key = __brev(path[i]) >> (32 - depth);
    r[i].margin = best[i];
    if (TRACK) {
      const uint32_t lvl = info[i] >> kPathLevelShift;
      r[i].ord = info[i] & ((1u << kPathLevelShift) - 1u);
      // the path's leading `lvl` bits are the index of the selected vertex inside its level
      r[i].vertex = FERN ? lvl : ((1u << lvl) - 1u) + (lvl == 0 ? 0u : path[i] >> (uint32_t(depth) - lvl));
    } else {
      r[i].vertex = 0;
      r[i].ord = 0;
    }
  }
}

// walk_paths for the forward pass over float data known to be "plain": every feature and threshold finite and no
// threshold equal to -0.0. Then t = thr - x carries everything the walk needs -- |t| is |margin| and the sign bit of t
// is the decision (x > thr  <=>  t < 0; t is +0.0 whenever x == thr, and never NaN) -- so a level costs one
// subtraction, one funnel shift that appends the sign bit to the path, and one minimum. The path is kept as a 1-based
// heap index (root = 1, child = 2 i + decision), so that the address of the next vertex is one shift-add: for trees
// node(i, at) is called with that 1-based index (the caller passes a table pointer moved back by one vertex), for
// ferns with the level. At the end heap = 2^depth + path and the leaf key is brev(heap) >> (32 - depth): the marker
// bit falls off. r.margin holds |margin|.
template <bool FERN, int N, typename NodeFn, typename FeatureFn>
__device__ __forceinline__ void walk_paths_plain(int depth, NodeFn node, FeatureFn feature, WalkResult<float> (&r)[N]) {
  uint32_t heap[N];
  float best_abs[N];
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const Node<float> n = node(i, FERN ? 0u : 1u);
    const float t = n.thr - feature(i, int(n.ord));
    heap[i] = __builtin_amdgcn_alignbit(1u, __float_as_uint(t), 31);  // 2 | sign(t)
    best_abs[i] = ht_abs(t);
  }
  for (int lvl = 1; lvl < depth; ++lvl) {
    Node<float> n[N];
#pragma unroll
    for (int i = 0; i < N; ++i) n[i] = node(i, FERN ? uint32_t(lvl) : heap[i]);
    float t[N];
#pragma unroll
    for (int i = 0; i < N; ++i) t[i] = n[i].thr - feature(i, int(n[i].ord));
#pragma unroll
    for (int i = 0; i < N; ++i) {
      // min of two non-negative, never-NaN values as the median with zero: one instruction, where fminf would first
      // quiet its operands
      best_abs[i] = __builtin_amdgcn_fmed3f(best_abs[i], ht_abs(t[i]), 0.f);
      heap[i] = __builtin_amdgcn_alignbit(heap[i], __float_as_uint(t[i]), 31);  // (heap << 1) | sign(t)
    }
  }
#pragma unroll
  for (int i = 0; i < N; ++i) {
    r[i].key = __brev(heap[i]) >> (32 - depth);
    r[i].vertex = 0;
    r[i].ord = 0;
    r[i].margin = best_abs[i];
  }
}

// walk_paths_plain for the backward pass: beside the path the walk carries t = thr - x of the selected vertex (the
// signed margin is -t, its magnitude |t|) and one word, level << 26 | ordinal (see walk_paths). Same 1-based heap
// index and the same contract for node(i, at) as walk_paths_plain. At the end heap = 2^depth + path:
//   leaf key            brev(heap) >> (32 - depth)           (the marker bit falls off)
//   selected vertex     (heap >> (depth - level)) - 1        (0-based heap index; ferns: the level itself)
struct TrackedPath {
  uint32_t heap;
  float t;
  uint32_t info;
  __device__ __forceinline__ uint32_t key(int depth) const { return __brev(heap) >> (32 - depth); }
  __device__ __forceinline__ uint32_t level() const { return info >> kPathLevelShift; }
  __device__ __forceinline__ uint32_t ordinal() const { return info & ((1u << kPathLevelShift) - 1u); }
  template <bool FERN>
  __device__ __forceinline__ uint32_t vertex(int depth) const {
    return FERN ? level() : (heap >> (uint32_t(depth) - level())) - 1u;
  }
};
template <bool FERN, int N, typename NodeFn, typename FeatureFn>
__device__ __forceinline__ void walk_paths_plain_tracked(int depth, NodeFn node, FeatureFn feature,
                                                         TrackedPath (&r)[N]) {
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const Node<float> n = node(i, FERN ? 0u : 1u);
    const float t = n.thr - feature(i, int(n.ord));
    r[i].heap = __builtin_amdgcn_alignbit(1u, __float_as_uint(t), 31);  // 2 | sign(t)
    r[i].t = t;
    r[i].info = uint32_t(n.ord);
  }
  for (int lvl = 1; lvl < depth; ++lvl) {
    const uint32_t lvl_tag = uint32_t(lvl) << kPathLevelShift;  // wave uniform
    Node<float> n[N];
#pragma unroll
    for (int i = 0; i < N; ++i) n[i] = node(i, FERN ? uint32_t(lvl) : r[i].heap);
    float t[N];
#pragma unroll
    for (int i = 0; i < N; ++i) t[i] = n[i].thr - feature(i, int(n[i].ord));
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const bool closer = ht_abs(t[i]) < ht_abs(r[i].t);
      r[i].t = closer ? t[i] : r[i].t;
      r[i].info = closer ? (lvl_tag | uint32_t(n[i].ord)) : r[i].info;
      r[i].heap = __builtin_amdgcn_alignbit(r[i].heap, __float_as_uint(t[i]), 31);  // (heap << 1) | sign(t)
    }
  }
}

// Whether a value keeps a walk "plain" in the sense of walk_paths_plain.
__device__ __forceinline__ bool plain_feature(float v) { return ht_abs(v) < __builtin_inff(); }
__device__ __forceinline__ bool plain_threshold(float v) {
  return ht_abs(v) < __builtin_inff() && __float_as_uint(v) != 0x80000000u;
}
__device__ __forceinline__ bool plain_feature(double) { return false; }
__device__ __forceinline__ bool plain_threshold(double) { return false; }

// Single walk over separate threshold / ordinal arrays (used where the vertices are not packed).
// `node(i)` returns (threshold, ordinal) of decision i; `feature(f)` returns this sample's value of feature f.
template <typename Real, bool FERN, typename NodeFn, typename FeatureFn>
__device__ __forceinline__ WalkResult<Real> walk(int depth, NodeFn node, FeatureFn feature) {
  WalkResult<Real> r;
  uint32_t v = 0;
  r.key = 0;
  r.vertex = 0;
  r.ord = 0;
  r.margin = Real(0);
  Real best_abs = Real(0);
  for (int lvl = 0; lvl < depth; ++lvl) {
    const uint32_t at = FERN ? uint32_t(lvl) : v;
    Real th;
    int o;
    node(at, th, o);
    const Real m = feature(o) - th;
    const uint32_t bit = (m > Real(0)) ? 1u : 0u;
    const Real a = ht_abs(m);
    if (lvl == 0 || a < best_abs) {
      best_abs = a;
      r.margin = m;
      r.vertex = at;
      r.ord = uint32_t(o);
    }
    r.key |= bit << lvl;
    v = 2u * v + 1u + bit;
  }
  return r;
}

}  // namespace ht
