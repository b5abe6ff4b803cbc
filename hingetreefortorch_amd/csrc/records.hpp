// Walk records: what the backward pass needs to know about every (tree, sample) pair, stored tree major
// (index t * S + s) so that a tree-stationary kernel streams them and a sample tile reads short contiguous runs.
//
// They are written either by the backward's own records kernel or, on the training path, by the forward pass while it
// has the walk results in registers anyway (the backward then does not walk again). The part a forward pass hands to
// a later backward is `saved` (10 bytes per pair in the compact form); c is scratch of the backward pass.
#pragma once
#include "common.hpp"

namespace ht {

// COMPACT (depth <= 16 and F <= 65536): key | vertex << 16 in one word, ordinal in 16 bits.
template <typename Real, bool COMPACT>
struct Records {
  uint32_t *a;    // COMPACT: key | vertex << 16      else: key
  uint32_t *b;    // COMPACT: unused                  else: vertex
  void *ordinal;  // COMPACT: uint16_t[]              else: uint32_t[]
  Real *margin;
  Real *c;        // sign(margin) * sum_m w * g, filled by the tree kernel

  __device__ __forceinline__ void put(long long at, uint32_t key, uint32_t vertex, uint32_t ord, Real m) const {
    if (COMPACT) {
      a[at] = key | (vertex << 16);
      static_cast<uint16_t *>(ordinal)[at] = uint16_t(ord);
    } else {
      a[at] = key;
      b[at] = vertex;
      static_cast<uint32_t *>(ordinal)[at] = ord;
    }
    margin[at] = m;
  }
  __device__ __forceinline__ uint32_t key(long long at) const { return COMPACT ? (a[at] & 0xffffu) : a[at]; }
  __device__ __forceinline__ uint32_t vertex(long long at) const { return COMPACT ? (a[at] >> 16) : b[at]; }
  __device__ __forceinline__ uint32_t ord(long long at) const {
    return COMPACT ? uint32_t(static_cast<const uint16_t *>(ordinal)[at]) : static_cast<const uint32_t *>(ordinal)[at];
  }
};

static inline bool compact_ok(const ForestDims &d) { return d.depth <= 16 && d.F <= 65536; }

// Bytes of the saved part (key, vertex, ordinal, margin) ...
template <typename Real>
static inline size_t records_saved_bytes(const ForestDims &d) {
  const size_t n = size_t(d.T) * size_t(d.S);
  if (compact_ok(d)) return align_up(n * 4, 256) + align_up(n * 2, 256) + align_up(n * sizeof(Real), 256);
  return 3 * align_up(n * 4, 256) + align_up(n * sizeof(Real), 256);
}
// ... and of the c scratch.
template <typename Real>
static inline size_t records_scratch_bytes(const ForestDims &d) {
  return align_up(size_t(d.T) * size_t(d.S) * sizeof(Real), 256);
}

template <typename Real, bool COMPACT>
static inline Records<Real, COMPACT> carve_records(const ForestDims &d, void *saved, void *scratch) {
  const size_t n = size_t(d.T) * size_t(d.S);
  unsigned char *p = static_cast<unsigned char *>(saved);
  Records<Real, COMPACT> r;
  r.a = reinterpret_cast<uint32_t *>(p);
  p += align_up(n * 4, 256);
  r.b = nullptr;
  if (!COMPACT) {
    r.b = reinterpret_cast<uint32_t *>(p);
    p += align_up(n * 4, 256);
  }
  r.ordinal = p;
  p += align_up(n * (COMPACT ? 2 : 4), 256);
  r.margin = reinterpret_cast<Real *>(p);
  r.c = static_cast<Real *>(scratch);
  return r;
}

}  // namespace ht
