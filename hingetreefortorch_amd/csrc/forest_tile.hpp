// Sample tile shared by the forest kernels.
//
// A workgroup owns BT consecutive samples (a sample is one (batch row, inner position) pair) and keeps all F features
// of them in LDS, feature major: xs[f * BT + j]. With lane = sample, a gather of *different* features by different
// lanes touches bank (j mod 32) only, so the data-dependent reads of the walk never conflict.
#pragma once
#include "common.hpp"
#include "walk.hpp"

namespace ht {

// Largest tile width whose feature-major copy fits the LDS budget left after `reserve` bytes; 0 if even 8 do not fit.
template <typename Real>
static inline int pick_tile(int F, size_t reserve) {
  const int candidates[4] = {64, 32, 16, 8};
  for (int bt : candidates)
    if (size_t(F) * bt * sizeof(Real) + reserve <= size_t(kLdsBytes)) return bt;
  return 0;
}

// Cooperative load of the tile starting at sample s0. NT must be a multiple of BT, so a thread always serves the
// same sample j and only its feature index advances. With K == 1 a sample's features are contiguous: each lane then
// takes four of them per load, and a wavefront walks along its own span of every row (16-byte chunks
// wave * CPW ... (wave + 1) * CPW), so the 128-byte lines of a row are requested by consecutive loads of one wavefront
// and reach L2 as one request each, rather than once from each of four wavefronts.
template <typename Real, int BT, int NT>
__device__ __forceinline__ void load_tile(Real *xs, const Real *__restrict__ x, const ForestDims &d, long long s0,
                                          const FeatureNorm<Real> norm = FeatureNorm<Real>()) {
  typedef Real Vec4 __attribute__((ext_vector_type(4)));
  const int j = threadIdx.x % BT;
  const long long s = s0 + j;
  const bool live = s < d.S;
  const long long base = live ? (s / d.K) * d.FK + (s % d.K) : 0;
  if (d.K == 1 && d.F % 4 == 0 && reinterpret_cast<uintptr_t>(x) % sizeof(Vec4) == 0) {
    constexpr int G = NT / BT;                           // chunk slots of the workgroup per step
    constexpr int R = BT >= kWave ? 1 : kWave / BT;      // ... of which a wavefront holds R
    constexpr int W = G / R > 0 ? G / R : 1;             // spans
    const int slot = threadIdx.x / BT, span = slot / R, r = slot % R;
    const int chunks = d.F / 4;
    const int cpw = ((chunks + W - 1) / W + R - 1) / R * R;  // chunks per span, a multiple of R
    const int c_end = min(chunks, (span + 1) * cpw);
    for (int c = span * cpw + r; c < c_end; c += R) {
      Vec4 v = {Real(0), Real(0), Real(0), Real(0)};
      if (live) v = *reinterpret_cast<const Vec4 *>(x + base + 4 * c);
      if (norm.mean != nullptr && live) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = (v[i] - norm.mean[4 * c + i]) * norm.rstd[4 * c + i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) xs[(4 * c + i) * BT + j] = v[i];
    }
    return;
  }
  for (int f = threadIdx.x / BT; f < d.F; f += NT / BT) {
    Real v = live ? x[base + (long long)f * d.K] : Real(0);
    if (norm.mean != nullptr && live) v = (v - norm.mean[f]) * norm.rstd[f];
    xs[f * BT + j] = v;
  }
}

// Flat offset of element (sample s, tree t, output m) of the [B, T, K, M] output / upstream-gradient tensors.
__device__ __forceinline__ long long out_offset(const ForestDims &d, long long s, int t, int m) {
  const long long b = s / d.K, k = s % d.K;
  return ((b * d.T + t) * d.K + k) * d.M + m;
}

}  // namespace ht
