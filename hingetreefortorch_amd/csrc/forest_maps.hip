// Leaf map, margin map, reachability, ordinal range and the zero-fill helper.
#include "forest_tile.hpp"

namespace ht {
namespace {

// Same tile walk as the forward; each (sample, tree) pair writes its observables directly.
template <typename Real, bool FERN, int BT, bool XLDS>
__global__ __launch_bounds__(kForestThreads) void maps_kernel(ForestDims d, const Real *__restrict__ x,
                                                              const Real *__restrict__ thr,
                                                              const int64_t *__restrict__ ord, int64_t *leafmap,
                                                              Real *margins, int64_t *ordinals,
                                                              unsigned long long *reach, uint16_t *keys,
                                                              int trees_per_block) {
  constexpr int NT = kForestThreads;
  constexpr int TC = NT / BT;
  extern __shared__ __align__(16) unsigned char smem[];
  Real *xs = reinterpret_cast<Real *>(smem);
  const long long s0 = (long long)blockIdx.x * BT;
  if (XLDS) {
    load_tile<Real, BT, NT>(xs, x, d, s0);
    __syncthreads();
  }
  const int j = threadIdx.x % BT, tt = threadIdx.x / BT;
  const long long s = s0 + j;
  if (s >= d.S) return;
  const long long b = s / d.K, k = s % d.K;
  const long long xbase = b * d.FK + k;
  const int t_begin = blockIdx.y * trees_per_block;
  const int t_end = min(d.T, t_begin + trees_per_block);
  for (int t = t_begin + tt; t < t_end; t += TC) {
    const Real *th = thr + (long long)t * d.V;
    const int64_t *od = ord + (long long)t * d.V;
    auto node = [&](uint32_t at, Real &tv, int &ov) { tv = th[at]; ov = clamp_ordinal(od[at], d.F); };
    WalkResult<Real> r;
    if (XLDS)
      r = walk<Real, FERN>(d.depth, node, [&](int f) { return xs[f * BT + j]; });
    else
      r = walk<Real, FERN>(d.depth, node, [&](int f) { return x[xbase + (long long)f * d.K]; });
    const long long at = (b * d.T + t) * d.K + k;
    if (leafmap) leafmap[at] = (int64_t)r.key;
    if (margins) margins[at] = r.margin;
    if (ordinals) ordinals[at] = od[r.vertex];
    if (keys)
      keys[(long long)t * d.S + s] = (uint16_t)r.key;
    else if (reach)
      atomicAdd(reach + (long long)t * d.L + r.key, 1ull);
  }
}

// Reachability as a histogram: the walk stores each pair's 16-bit leaf key tree-major, and here one workgroup counts a
// stretch of one tree's keys in LDS and adds its non-zero counters to the tree's row. A global atomic per pair, the
// other way to count, runs several times longer once a launch holds millions of pairs.
constexpr int kReachThreads = 256;

__global__ __launch_bounds__(kReachThreads) void reach_histogram_kernel(const uint16_t *__restrict__ keys, long long S,
                                                                        int L, long long per_part,
                                                                        unsigned long long *reach) {
  extern __shared__ __align__(16) unsigned char smem[];
  uint32_t *count = reinterpret_cast<uint32_t *>(smem);
  for (int l = threadIdx.x; l < L; l += kReachThreads) count[l] = 0u;
  __syncthreads();
  const int t = blockIdx.x;
  const uint16_t *row = keys + (long long)t * S;
  const long long s0 = (long long)blockIdx.y * per_part;
  const long long s1 = s0 + per_part < S ? s0 + per_part : S;
  if ((S & 7) == 0) {  // per_part is a multiple of 8, so every stretch of every tree starts on 16 bytes
    for (long long s = s0 + threadIdx.x * 8; s < s1; s += kReachThreads * 8) {
      const uint4 v = *reinterpret_cast<const uint4 *>(row + s);
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        atomicAdd(count + (w[i] & 0xffffu), 1u);
        atomicAdd(count + (w[i] >> 16), 1u);
      }
    }
  } else {
    for (long long s = s0 + threadIdx.x; s < s1; s += kReachThreads) atomicAdd(count + row[s], 1u);
  }
  __syncthreads();
  unsigned long long *dst = reach + (long long)t * L;
  for (int l = threadIdx.x; l < L; l += kReachThreads) {
    const uint32_t c = count[l];
    if (c) atomicAdd(dst + l, (unsigned long long)c);
  }
}

// The histogram needs 16-bit keys and a tree's counters in LDS, and pays off once there are enough pairs and a tree
// sees more samples than it has counters to clear and flush.
inline bool reach_by_histogram(const ForestDims &d) {
  return d.L <= 65536 && size_t(d.L) * 4 <= kLdsBytes && d.S * (long long)d.T >= (1 << 16) && d.S >= 2LL * d.L;
}

template <typename Real, bool FERN, int BT, bool XLDS>
int launch_maps(const ForestDims &d, const Real *x, const Real *thr, const int64_t *ord, int64_t *leafmap, Real *margins,
                int64_t *ordinals, int64_t *reach, uint16_t *keys, hipStream_t stream) {
  constexpr int TC = kForestThreads / BT;
  const size_t lds = XLDS ? size_t(d.F) * BT * sizeof(Real) : 0;
  const long long tiles = (d.S + BT - 1) / BT;
  const int passes = (d.T + TC - 1) / TC;
  long long want = tiles >= 512 ? 1 : (512 + tiles - 1) / tiles;
  const int split = int(want < passes ? want : passes);
  const int trees_per_block = ((passes + split - 1) / split) * TC;
  const int gy = (d.T + trees_per_block - 1) / trees_per_block;
  if (tiles > 0x7fffffffLL) return fail(HT_ERR_RUNTIME, "Error: too many sample tiles for one launch.");
  auto kernel = maps_kernel<Real, FERN, BT, XLDS>;
  HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(kernel)));
  hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)gy), dim3(kForestThreads), lds, stream, d, x, thr, ord,
                     leafmap, margins, ordinals, reinterpret_cast<unsigned long long *>(reach), keys,
                     trees_per_block);
  HT_LAUNCH_CHECK("forest maps");
  return HT_OK;
}

template <typename Real, bool FERN>
int dispatch_maps(const ForestDims &d, const Real *x, const Real *thr, const int64_t *ord, int64_t *leafmap,
                  Real *margins, int64_t *ordinals, int64_t *reach, uint16_t *keys, hipStream_t stream) {
  switch (pick_tile<Real>(d.F, 1024)) {
    case 64: return launch_maps<Real, FERN, 64, true>(d, x, thr, ord, leafmap, margins, ordinals, reach, keys, stream);
    case 32: return launch_maps<Real, FERN, 32, true>(d, x, thr, ord, leafmap, margins, ordinals, reach, keys, stream);
    case 16: return launch_maps<Real, FERN, 16, true>(d, x, thr, ord, leafmap, margins, ordinals, reach, keys, stream);
    case 8: return launch_maps<Real, FERN, 8, true>(d, x, thr, ord, leafmap, margins, ordinals, reach, keys, stream);
    default: return launch_maps<Real, FERN, 64, false>(d, x, thr, ord, leafmap, margins, ordinals, reach, keys, stream);
  }
}

// One store per thread with the blocks in address order: on this part that streams to HBM at ~6.9 TB/s, where a
// grid-stride loop over the same range reaches ~4.2 TB/s.
__global__ __launch_bounds__(256) void zero_kernel(uint32_t *p, size_t words) {
  const size_t i = (size_t(blockIdx.x) * blockDim.x + threadIdx.x) * 4;
  if (i + 4 <= words && (reinterpret_cast<uintptr_t>(p) & 15) == 0) {
    *reinterpret_cast<uint4 *>(p + i) = make_uint4(0u, 0u, 0u, 0u);
  } else {
    for (size_t k = i; k < words && k < i + 4; ++k) p[k] = 0u;
  }
}

__global__ void zero_tail_kernel(unsigned char *p, size_t bytes) {
  if (threadIdx.x < bytes) p[threadIdx.x] = 0;
}

__global__ void minmax_init_kernel(long long *mm) {
  mm[0] = 0x7fffffffffffffffLL;
  mm[1] = -0x7fffffffffffffffLL - 1;
}

__global__ __launch_bounds__(256) void minmax_kernel(const long long *__restrict__ v, long long n, long long *mm) {
  long long lo = 0x7fffffffffffffffLL, hi = -0x7fffffffffffffffLL - 1;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
    const long long a = v[i];
    lo = a < lo ? a : lo;
    hi = a > hi ? a : hi;
  }
  for (int off = 32; off > 0; off >>= 1) {
    const long long lo2 = __shfl_xor(lo, off, kWave), hi2 = __shfl_xor(hi, off, kWave);
    lo = lo2 < lo ? lo2 : lo;
    hi = hi2 > hi ? hi2 : hi;
  }
  if ((threadIdx.x & (kWave - 1)) == 0) {
    atomicMin(mm, lo);
    atomicMax(mm + 1, hi);
  }
}

}  // namespace

int zero_fill(void *p, size_t bytes, hipStream_t stream) {
  if (bytes == 0) return HT_OK;
  const size_t words = bytes / 4, tail = bytes % 4;
  if (words) {
    const size_t blocks = (words + 1023) / 1024;
    if (blocks > 0x7fffffffull) return fail(HT_ERR_RUNTIME, "Error: buffer too large to clear in one launch.");
    hipLaunchKernelGGL(zero_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, static_cast<uint32_t *>(p), words);
    HT_LAUNCH_CHECK("zero fill");
  }
  if (tail) {
    hipLaunchKernelGGL(zero_tail_kernel, dim3(1), dim3(4), 0, stream, static_cast<unsigned char *>(p) + words * 4, tail);
    HT_LAUNCH_CHECK("zero fill tail");
  }
  return HT_OK;
}

int ordinal_range(const int64_t *ord, int64_t n, int64_t *minmax, hipStream_t stream) {
  hipLaunchKernelGGL(minmax_init_kernel, dim3(1), dim3(1), 0, stream, reinterpret_cast<long long *>(minmax));
  HT_LAUNCH_CHECK("ordinal range init");
  if (n > 0) {
    long long blocks = (n + 255) / 256;
    if (blocks > 1024) blocks = 1024;
    hipLaunchKernelGGL(minmax_kernel, dim3((unsigned)blocks), dim3(256), 0, stream,
                       reinterpret_cast<const long long *>(ord), (long long)n, reinterpret_cast<long long *>(minmax));
    HT_LAUNCH_CHECK("ordinal range");
  }
  return HT_OK;
}

// Workspace: the 16-bit leaf keys that let reachability run as a histogram, then the packed vertices that let every
// map run on the forward's row kernel walk. The call works without either (or with less), slower.
static size_t reach_keys_bytes(const ForestDims &d) {
  return reach_by_histogram(d) ? align_up(size_t(d.S) * d.T * sizeof(uint16_t), 256) : 0;
}
template <typename Real>
size_t forest_maps_workspace(const ForestDims &d, bool want_reach) {
  if (d.S == 0 || d.T == 0) return 0;
  return (want_reach ? reach_keys_bytes(d) : 0) + forest_maps_rows_workspace<Real>(d);
}

static int launch_reach_histogram(const ForestDims &d, const uint16_t *keys, int64_t *reach, hipStream_t stream) {
  // enough workgroups to fill the part, each with a stretch of keys that is worth its counter flush
  long long parts = (2048 + d.T - 1) / d.T;
  const long long most = (d.S + 4LL * d.L - 1) / (4LL * d.L);
  if (parts > most) parts = most;
  if (parts < 1) parts = 1;
  if (parts > 65535) parts = 65535;
  long long per_part = (d.S + parts - 1) / parts;
  per_part = (per_part + 7) / 8 * 8;
  parts = (d.S + per_part - 1) / per_part;
  const size_t lds = size_t(d.L) * 4;
  HT_HIP_CHECK(grant_lds(reinterpret_cast<const void *>(reach_histogram_kernel)));
  hipLaunchKernelGGL(reach_histogram_kernel, dim3((unsigned)d.T, (unsigned)parts), dim3(kReachThreads), lds, stream,
                     keys, (long long)d.S, d.L, per_part, reinterpret_cast<unsigned long long *>(reach));
  HT_LAUNCH_CHECK("reachability histogram");
  return HT_OK;
}

template <typename Real>
int forest_maps(const ForestDims &d, bool fern, const Real *x, const Real *thr, const int64_t *ord, int64_t *leafmap,
                Real *margins, int64_t *ordinals, int64_t *reach, void *workspace, size_t workspace_bytes,
                hipStream_t stream) {
  int rc;
  if (reach && (rc = zero_fill(reach, size_t(d.T) * d.L * sizeof(int64_t), stream)) != HT_OK) return rc;
  if (d.S == 0 || d.T == 0) return HT_OK;
  const bool aligned = workspace && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0;
  const size_t key_bytes = reach_keys_bytes(d), row_bytes = forest_maps_rows_workspace<Real>(d);
  // the row kernel's walk: wherever its packed vertices have room in the workspace -- and, for reachability, the keys
  // of the histogram as well (its other form, one global atomic per pair, stays with the plain kernel below)
  const bool keys_fit = key_bytes != 0 && aligned && workspace_bytes >= key_bytes;
  const size_t rows_at = reach ? key_bytes : 0;
  if (row_bytes != 0 && aligned && workspace_bytes >= rows_at + row_bytes && (!reach || keys_fit)) {
    uint16_t *keys = reach ? static_cast<uint16_t *>(workspace) : nullptr;
    void *vertices = static_cast<unsigned char *>(workspace) + rows_at;
    if ((rc = forest_maps_rows<Real>(d, fern, x, thr, ord, leafmap, keys, margins, ordinals, vertices, stream)) != HT_OK)
      return rc;
    return reach ? launch_reach_histogram(d, keys, reach, stream) : HT_OK;
  }
  uint16_t *keys = (reach && keys_fit) ? static_cast<uint16_t *>(workspace) : nullptr;
  rc = fern ? dispatch_maps<Real, true>(d, x, thr, ord, leafmap, margins, ordinals, reach, keys, stream)
            : dispatch_maps<Real, false>(d, x, thr, ord, leafmap, margins, ordinals, reach, keys, stream);
  if (rc != HT_OK || !keys) return rc;
  return launch_reach_histogram(d, keys, reach, stream);
}

template size_t forest_maps_workspace<float>(const ForestDims &, bool);
template size_t forest_maps_workspace<double>(const ForestDims &, bool);
template int forest_maps<float>(const ForestDims &, bool, const float *, const float *, const int64_t *, int64_t *,
                                float *, int64_t *, int64_t *, void *, size_t, hipStream_t);
template int forest_maps<double>(const ForestDims &, bool, const double *, const double *, const int64_t *, int64_t *,
                                 double *, int64_t *, int64_t *, void *, size_t, hipStream_t);

}  // namespace ht
