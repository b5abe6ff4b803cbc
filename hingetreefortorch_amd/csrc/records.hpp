// Walk records: what the backward pass needs to know about every (tree, sample) pair, stored tree major
// (index t * S + s) so that a tree-stationary kernel streams them and a sample tile reads short contiguous runs.
//
// They are written either by the backward's own records kernel or, on the training path, by the forward pass while it
// has the walk results in registers anyway (the backward then does not walk again). The part a forward pass hands to
// a later backward is `saved` (10 bytes per pair in the compact form); c is scratch of the backward pass.
#pragma once
#include "common.hpp"

namespace ht {

// COMPACT (depth <= 16 and F <= 65536): key | vertex << vshift in one word. Where depth + depth + bits(F) <= 32 the
// selected ordinal rides in the same word (ord << oshift, "packed": 8 bytes per pair instead of 10 and one store
// fewer per walk); otherwise vshift = 16 and the ordinal has its own 16-bit array.
// A bound on |margin| over all pairs rides along with the saved part: whoever writes the records keeps a running
// maximum per lane and publishes it with one atomic per wavefront into kBoundSlots slots (spread by workgroup, because
// thousands of atomics on one address serialise in L2); the deterministic backward folds the slots when it picks its
// fixed-point scale, instead of reading all margins again. The slots are cleared by the vertex-packing pre-pass that
// precedes every kernel that writes records.
constexpr int kBoundSlots = 1024;

// Running bound on |v| (NaN counts as +inf) ...
__device__ __forceinline__ void bound_take(float &m, float v) {
  const float a = __builtin_fabsf(v);
  if (!(a <= m)) m = (a != a) ? __builtin_inff() : a;
}
__device__ __forceinline__ void bound_take(double &m, double v) {
  const double a = __builtin_fabs(v);
  if (!(a <= m)) m = (a != a) ? double(__builtin_inff()) : a;
}
// ... and its maximum over the wavefront into slot `which` (as the bit pattern of a non-negative double, which orders
// like the value).
__device__ __forceinline__ void bound_publish(double m, unsigned long long *slots, unsigned which) {
  for (int off = 32; off > 0; off >>= 1) {
    const double o = __shfl_xor(m, off, 64);
    if (!(o <= m)) m = o;
  }
  if ((threadIdx.x & 63u) == 0 && m > 0.0) atomicMax(slots + which, (unsigned long long)__double_as_longlong(m));
}

// The same bound for kernels that cannot spare the instructions (the forward pass takes one per walk): the magnitude
// bits of a float order like its magnitude, with every NaN above infinity, so the running maximum is one AND and one
// integer MAX per value; a double contributes its upper word with the lower word taken as all ones (a bound is all
// that is needed). margin_bound_value turns the bits back into a double, NaN patterns into +inf.
struct MarginBits {
  uint32_t bits = 0;
  __device__ __forceinline__ void take(float v) { bits = max(bits, __float_as_uint(v) & 0x7fffffffu); }
  __device__ __forceinline__ void take(double v) { bits = max(bits, uint32_t(__double2hiint(v)) & 0x7fffffffu); }
  // for a value whose sign bit is already clear
  __device__ __forceinline__ void take_abs(float a) { bits = max(bits, __float_as_uint(a)); }
  __device__ __forceinline__ void take_abs(double a) { bits = max(bits, uint32_t(__double2hiint(a))); }
};
template <typename Real>
__device__ __forceinline__ double margin_bound_value(uint32_t bits) {
  if (sizeof(Real) == 4) return bits >= 0x7f800000u ? double(__builtin_inff()) : double(__uint_as_float(bits));
  return bits >= 0x7ff00000u ? double(__builtin_inff()) : __hiloint2double(int(bits), -1);
}

template <typename Real, bool COMPACT>
struct Records {
  uint32_t *a;    // COMPACT: key | vertex << vshift [| ord << oshift]      else: key
  uint32_t *b;    // COMPACT: unused                                        else: vertex
  void *ordinal;  // COMPACT: uint16_t[] unless packed                      else: uint32_t[]
  Real *margin;
  Real *c;        // sign(margin) * sum_m w * g, filled by the tree kernel
  unsigned long long *bound;  // kBoundSlots slots: max |margin| over all pairs (see above)
  int vshift, oshift;  // COMPACT only; oshift == 0: ordinals in their own array

  __device__ __forceinline__ uint32_t key_mask() const { return COMPACT ? ((1u << vshift) - 1u) : 0xffffffffu; }
  __device__ __forceinline__ void put(long long at, uint32_t key, uint32_t vertex, uint32_t ord, Real m) const {
    if (COMPACT) {
      if (oshift) {
        __builtin_nontemporal_store(key | (vertex << vshift) | (ord << oshift), a + at);
      } else {
        __builtin_nontemporal_store(key | (vertex << vshift), a + at);
        static_cast<uint16_t *>(ordinal)[at] = uint16_t(ord);
      }
    } else {
      a[at] = key;
      b[at] = vertex;
      static_cast<uint32_t *>(ordinal)[at] = ord;
    }
    __builtin_nontemporal_store(m, margin + at);
  }
  __device__ __forceinline__ uint32_t key(long long at) const { return COMPACT ? (a[at] & key_mask()) : a[at]; }
  __device__ __forceinline__ uint32_t vertex(long long at) const {
    return COMPACT ? ((a[at] >> vshift) & key_mask()) : b[at];
  }
  __device__ __forceinline__ uint32_t ord(long long at) const {
    if (COMPACT) return oshift ? (a[at] >> oshift) : uint32_t(static_cast<const uint16_t *>(ordinal)[at]);
    return static_cast<const uint32_t *>(ordinal)[at];
  }
};

static inline bool compact_ok(const ForestDims &d) { return d.depth <= 16 && d.F <= 65536; }
// ... and the ordinal fits beside key and vertex
static inline bool packed_ok(const ForestDims &d) {
  int fbits = 0;
  while ((1ll << fbits) < d.F) ++fbits;
  return compact_ok(d) && 2 * d.depth + fbits <= 32;
}

// Bytes of the saved part (key, vertex, ordinal, margin, the bound slots) ...
constexpr size_t kBoundBytes = size_t(kBoundSlots) * sizeof(unsigned long long);
template <typename Real>
static inline size_t records_saved_bytes(const ForestDims &d) {
  const size_t n = size_t(d.T) * size_t(d.S);
  if (packed_ok(d)) return align_up(n * 4, 256) + align_up(n * sizeof(Real), 256) + kBoundBytes;
  if (compact_ok(d)) return align_up(n * 4, 256) + align_up(n * 2, 256) + align_up(n * sizeof(Real), 256) + kBoundBytes;
  return 3 * align_up(n * 4, 256) + align_up(n * sizeof(Real), 256) + kBoundBytes;
}
// ... whose last kBoundBytes are the slots
template <typename Real>
static inline unsigned long long *records_bound_slots(const ForestDims &d, void *saved) {
  return reinterpret_cast<unsigned long long *>(static_cast<unsigned char *>(saved) + records_saved_bytes<Real>(d) -
                                                kBoundBytes);
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
  const bool packed = COMPACT && packed_ok(d);
  r.vshift = packed ? d.depth : 16;
  r.oshift = packed ? 2 * d.depth : 0;
  r.a = reinterpret_cast<uint32_t *>(p);
  p += align_up(n * 4, 256);
  r.b = nullptr;
  if (!COMPACT) {
    r.b = reinterpret_cast<uint32_t *>(p);
    p += align_up(n * 4, 256);
  }
  r.ordinal = p;
  if (!packed) p += align_up(n * (COMPACT ? 2 : 4), 256);
  r.margin = reinterpret_cast<Real *>(p);
  r.c = static_cast<Real *>(scratch);
  r.bound = records_bound_slots<Real>(d, saved);
  return r;
}

}  // namespace ht
