// Forest / fern backward: dX, dThresholds, dWeights.
//
// Atomic mode: one fused kernel. Same sample tile as the forward; per pass every (sample, tree) pair is walked once,
// the upstream gradient is read once with the thread index along its contiguous axis, dW is accumulated with one
// atomic per element, and the per-pair scalar c = sum_m w[t,leaf,m] * g[b,t,k,m] is reduced in LDS before the two
// scatter atomics (dX, dThr) are issued.
//
// Deterministic mode: the walk is done once by a tile kernel that writes (leaf, vertex, margin) records, then
//   * dX is owner-computes: one thread per sample adds its trees in index order (the reference CPU order);
//   * dThr / dW are owner-computes per tree: one wavefront per tree consumes its records in sample order and orders
//     colliding updates inside each group of 64 samples by lane, so no result depends on scheduling.
#include "forest_tile.hpp"

namespace ht {
namespace {

template <typename Real>
__device__ __forceinline__ void atomic_add(Real *p, Real v) {
  atomicAdd(p, v);
}

// ---------------------------------------------------------------------------------------------------------------
// atomic mode
// ---------------------------------------------------------------------------------------------------------------
template <typename Real, bool FERN, int BT, bool XLDS>
__global__ __launch_bounds__(kForestThreads) void backward_atomic_kernel(
    ForestDims d, const Real *__restrict__ x, const Real *__restrict__ thr, const int64_t *__restrict__ ord,
    const Real *__restrict__ w, const Real *__restrict__ gout, Real *__restrict__ dx, Real *__restrict__ dthr,
    Real *__restrict__ dw, int trees_per_block) {
  constexpr int NT = kForestThreads;
  constexpr int TC = NT / BT;
  extern __shared__ __align__(16) unsigned char smem[];
  Real *xs = reinterpret_cast<Real *>(smem);
  Real *r_margin = xs + (XLDS ? size_t(d.F) * BT : 0);
  Real *r_csum = r_margin + TC * BT;
  uint32_t *r_key = reinterpret_cast<uint32_t *>(r_csum + TC * BT);
  uint32_t *r_vertex = r_key + TC * BT;

  const long long s0 = (long long)blockIdx.x * BT;
  if (XLDS) {
    load_tile<Real, BT, NT>(xs, x, d, s0);
    __syncthreads();
  }
  const int j = threadIdx.x % BT, tt = threadIdx.x / BT;
  const long long s = s0 + j;
  const bool live = s < d.S;
  const long long xbase = live ? (s / d.K) * d.FK + (s % d.K) : 0;
  const bool need_c = (dx != nullptr) || (dthr != nullptr);

  const int t_begin = blockIdx.y * trees_per_block;
  const int t_end = min(d.T, t_begin + trees_per_block);
  for (int tb = t_begin; tb < t_end; tb += TC) {
    const int t = tb + tt;
    const bool mine = t < t_end && live;
    if (mine) {
      const Real *th = thr + (long long)t * d.V;
      const int64_t *od = ord + (long long)t * d.V;
      auto node = [&](uint32_t at, Real &tv, int &ov) { tv = th[at]; ov = clamp_ordinal(od[at], d.F); };
      WalkResult<Real> r;
      if (XLDS)
        r = walk<Real, FERN>(d.depth, node, [&](int f) { return xs[f * BT + j]; });
      else
        r = walk<Real, FERN>(d.depth, node, [&](int f) { return x[xbase + (long long)f * d.K]; });
      r_margin[tt * BT + j] = r.margin;
      r_key[tt * BT + j] = r.key;
      r_vertex[tt * BT + j] = r.vertex;
    }
    r_csum[tt * BT + j] = Real(0);
    __syncthreads();

    const int nt = min(TC, t_end - tb);
    {
      const bool k1 = d.K == 1;
      const int row = k1 ? nt * d.M : BT * d.M;
      const int total = k1 ? BT * row : nt * row;
      for (int idx = threadIdx.x; idx < total; idx += NT) {
        const int hi = idx / row, r = idx - hi * row;
        const int lo = r / d.M, m = r - lo * d.M;
        const int jj = k1 ? hi : lo, t2 = k1 ? lo : hi;
        const long long ss = s0 + jj;
        if (ss < d.S) {
          const Real g = gout[out_offset(d, ss, tb + t2, m)];
          const uint32_t key = r_key[t2 * BT + jj];
          const long long wi = ((long long)(tb + t2) * d.L + key) * d.M + m;
          if (dw) atomic_add(dw + wi, ht_abs(r_margin[t2 * BT + jj]) * g);
          if (need_c) atomic_add(r_csum + t2 * BT + jj, w[wi] * g);
        }
      }
    }
    __syncthreads();

    if (mine && need_c) {
      const Real c = ht_sign(r_margin[tt * BT + j]) * r_csum[tt * BT + j];
      const uint32_t v = r_vertex[tt * BT + j];
      const long long o = clamp_ordinal(ord[(long long)t * d.V + v], d.F);
      if (dx) atomic_add(dx + xbase + o * d.K, c);
      if (dthr) atomic_add(dthr + (long long)t * d.V + v, -c);
    }
    __syncthreads();
  }
}

template <typename Real, bool FERN, int BT, bool XLDS>
int launch_backward_atomic(const ForestDims &d, const Real *x, const Real *thr, const int64_t *ord, const Real *w,
                           const Real *gout, Real *dx, Real *dthr, Real *dw, hipStream_t stream) {
  constexpr int TC = kForestThreads / BT;
  const size_t lds =
      (XLDS ? size_t(d.F) * BT * sizeof(Real) : 0) + size_t(TC) * BT * (2 * sizeof(Real) + 2 * sizeof(uint32_t));
  const long long tiles = (d.S + BT - 1) / BT;
  const int passes = (d.T + TC - 1) / TC;
  long long want = tiles >= 512 ? 1 : (512 + tiles - 1) / tiles;
  const int split = int(want < passes ? want : passes);
  const int trees_per_block = ((passes + split - 1) / split) * TC;
  const int gy = (d.T + trees_per_block - 1) / trees_per_block;
  if (tiles > 0x7fffffffLL) return fail(HT_ERR_RUNTIME, "Error: too many sample tiles for one launch.");
  auto kernel = backward_atomic_kernel<Real, FERN, BT, XLDS>;
  HT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   int(lds)));
  hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)gy), dim3(kForestThreads), lds, stream, d, x, thr, ord, w,
                     gout, dx, dthr, dw, trees_per_block);
  HT_LAUNCH_CHECK("forest backward (atomic)");
  return HT_OK;
}

template <typename Real, bool FERN>
int dispatch_backward_atomic(const ForestDims &d, const Real *x, const Real *thr, const int64_t *ord, const Real *w,
                             const Real *gout, Real *dx, Real *dthr, Real *dw, hipStream_t stream) {
  const size_t reserve = 32 * 1024;
  switch (pick_tile<Real>(d.F, reserve)) {
    case 64: return launch_backward_atomic<Real, FERN, 64, true>(d, x, thr, ord, w, gout, dx, dthr, dw, stream);
    case 32: return launch_backward_atomic<Real, FERN, 32, true>(d, x, thr, ord, w, gout, dx, dthr, dw, stream);
    case 16: return launch_backward_atomic<Real, FERN, 16, true>(d, x, thr, ord, w, gout, dx, dthr, dw, stream);
    case 8: return launch_backward_atomic<Real, FERN, 8, true>(d, x, thr, ord, w, gout, dx, dthr, dw, stream);
    default: return launch_backward_atomic<Real, FERN, 64, false>(d, x, thr, ord, w, gout, dx, dthr, dw, stream);
  }
}

// ---------------------------------------------------------------------------------------------------------------
// deterministic mode
// ---------------------------------------------------------------------------------------------------------------
// Walk records, tree major: rec[t * S + s].
template <typename Real>
struct Records {
  uint32_t *key;
  uint32_t *vertex;
  Real *margin;
};

template <typename Real>
size_t records_bytes(const ForestDims &d) {
  const size_t n = size_t(d.T) * size_t(d.S);
  return align_up(n * sizeof(uint32_t), 256) * 2 + align_up(n * sizeof(Real), 256);
}

template <typename Real>
Records<Real> carve_records(const ForestDims &d, void *ws) {
  const size_t n = size_t(d.T) * size_t(d.S);
  unsigned char *p = static_cast<unsigned char *>(ws);
  Records<Real> r;
  r.key = reinterpret_cast<uint32_t *>(p);
  p += align_up(n * sizeof(uint32_t), 256);
  r.vertex = reinterpret_cast<uint32_t *>(p);
  p += align_up(n * sizeof(uint32_t), 256);
  r.margin = reinterpret_cast<Real *>(p);
  return r;
}

template <typename Real, bool FERN, int BT, bool XLDS>
__global__ __launch_bounds__(kForestThreads) void records_kernel(ForestDims d, const Real *__restrict__ x,
                                                                 const Real *__restrict__ thr,
                                                                 const int64_t *__restrict__ ord, Records<Real> rec,
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
  const long long xbase = (s / d.K) * d.FK + (s % d.K);
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
    const long long at = (long long)t * d.S + s;
    rec.key[at] = r.key;
    rec.vertex[at] = r.vertex;
    rec.margin[at] = r.margin;
  }
}

template <typename Real, bool FERN, int BT, bool XLDS>
int launch_records(const ForestDims &d, const Real *x, const Real *thr, const int64_t *ord, Records<Real> rec,
                   hipStream_t stream) {
  constexpr int TC = kForestThreads / BT;
  const size_t lds = XLDS ? size_t(d.F) * BT * sizeof(Real) : 0;
  const long long tiles = (d.S + BT - 1) / BT;
  const int passes = (d.T + TC - 1) / TC;
  long long want = tiles >= 512 ? 1 : (512 + tiles - 1) / tiles;
  const int split = int(want < passes ? want : passes);
  const int trees_per_block = ((passes + split - 1) / split) * TC;
  const int gy = (d.T + trees_per_block - 1) / trees_per_block;
  if (tiles > 0x7fffffffLL) return fail(HT_ERR_RUNTIME, "Error: too many sample tiles for one launch.");
  auto kernel = records_kernel<Real, FERN, BT, XLDS>;
  HT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   int(lds)));
  hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)gy), dim3(kForestThreads), lds, stream, d, x, thr, ord,
                     rec, trees_per_block);
  HT_LAUNCH_CHECK("forest walk records");
  return HT_OK;
}

template <typename Real, bool FERN>
int dispatch_records(const ForestDims &d, const Real *x, const Real *thr, const int64_t *ord, Records<Real> rec,
                     hipStream_t stream) {
  switch (pick_tile<Real>(d.F, 1024)) {
    case 64: return launch_records<Real, FERN, 64, true>(d, x, thr, ord, rec, stream);
    case 32: return launch_records<Real, FERN, 32, true>(d, x, thr, ord, rec, stream);
    case 16: return launch_records<Real, FERN, 16, true>(d, x, thr, ord, rec, stream);
    case 8: return launch_records<Real, FERN, 8, true>(d, x, thr, ord, rec, stream);
    default: return launch_records<Real, FERN, 64, false>(d, x, thr, ord, rec, stream);
  }
}

// dX: thread per sample, trees in index order, one add per (tree, m) term straight into the owned cell: the same
// sequence of roundings as the reference CPU loop (hingetree.cpp:236-254).
template <typename Real>
__global__ __launch_bounds__(256) void det_dx_kernel(ForestDims d, const int64_t *__restrict__ ord,
                                                     const Real *__restrict__ w, const Real *__restrict__ gout,
                                                     Records<Real> rec, Real *dx) {
  const long long s = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (s >= d.S) return;
  const long long b = s / d.K, k = s % d.K;
  const long long xbase = b * d.FK + k;
  for (int t = 0; t < d.T; ++t) {
    const long long at = (long long)t * d.S + s;
    const uint32_t key = rec.key[at];
    const Real sg = ht_sign(rec.margin[at]);
    const long long o = clamp_ordinal(ord[(long long)t * d.V + rec.vertex[at]], d.F);
    const Real *wl = w + ((long long)t * d.L + key) * d.M;
    const Real *g = gout + ((b * d.T + t) * d.K + k) * d.M;
    Real *cell = dx + xbase + o * d.K;
    Real acc = *cell;
    for (int m = 0; m < d.M; ++m) acc += sg * wl[m] * g[m];
    *cell = acc;
  }
}

template <typename Real>
__device__ __forceinline__ Real wave_sum_fixed(Real v) {
  // butterfly with a fixed shape: the result depends only on the 64 lane values
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

// Adds v to *p. LDS: plain read-modify-write (the caller guarantees a single writer per address per step). Global:
// a returning atomic whose result is consumed, so the update has completed before the wavefront's next step.
template <typename Real, bool LDS_ACC>
__device__ __forceinline__ void ordered_add(Real *p, Real v) {
  if (LDS_ACC) {
    *p += v;
  } else {
    Real old = atomicAdd(p, v);
    asm volatile("" ::"v"(old));
  }
}

// dThr and dW of one tree by one wavefront, records consumed in sample order, 64 at a time.
//   dW  : lanes that hit the same leaf are ranked by lane; round r applies the rank-r lanes, so each cell receives
//         its terms in ascending sample order (the reference CPU order, hingetree.cpp:290-305).
//   dThr: for each distinct vertex in the group the member lanes' terms are summed by a fixed butterfly and the
//         leader lane adds the group sum to the vertex' accumulator.
template <typename Real, bool LDS_ACC>
__global__ __launch_bounds__(kWave) void det_tree_kernel(ForestDims d, const Real *__restrict__ w,
                                                         const Real *__restrict__ gout, Records<Real> rec, Real *dthr,
                                                         Real *dw) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int t = blockIdx.x;
  const int lane = threadIdx.x;
  const long long nW = (long long)d.L * d.M;
  Real *accW = nullptr, *accT = nullptr;
  if (LDS_ACC) {
    accW = reinterpret_cast<Real *>(smem);
    accT = accW + (dw ? nW : 0);
    if (dw)
      for (long long i = lane; i < nW; i += kWave) accW[i] = Real(0);
    if (dthr)
      for (int i = lane; i < d.V; i += kWave) accT[i] = Real(0);
    __syncthreads();
  } else {
    accW = dw ? dw + (long long)t * nW : nullptr;  // pre-zeroed by the host
    accT = dthr ? dthr + (long long)t * d.V : nullptr;
  }

  for (long long c0 = 0; c0 < d.S; c0 += kWave) {
    const long long s = c0 + lane;
    const bool live = s < d.S;
    uint32_t key = 0xffffffffu, v = 0xffffffffu;
    Real mg = Real(0);
    if (live) {
      const long long at = (long long)t * d.S + s;
      key = rec.key[at];
      v = rec.vertex[at];
      mg = rec.margin[at];
    }
    const long long goff = live ? out_offset(d, s, t, 0) : 0;
    const Real *g = gout + goff;

    if (dw) {
      int rank = 0;
      for (int l = 0; l < kWave; ++l) {
        const uint32_t other = __shfl(key, l, kWave);
        rank += (l < lane && other == key) ? 1 : 0;
      }
      if (!live) rank = -1;
      int rounds = rank;
      for (int off = 32; off > 0; off >>= 1) rounds = max(rounds, __shfl_xor(rounds, off, kWave));
      const Real a = ht_abs(mg);
      for (int r = 0; r <= rounds; ++r) {
        if (rank == r) {
          Real *cell = accW + (long long)key * d.M;
          for (int m = 0; m < d.M; ++m) ordered_add<Real, LDS_ACC>(cell + m, a * g[m]);
        }
        __syncthreads();
      }
    }

    if (dthr) {
      Real c = Real(0);
      if (live) {
        const Real *wl = w + ((long long)t * d.L + key) * d.M;
        for (int m = 0; m < d.M; ++m) c += wl[m] * g[m];
        c = -(ht_sign(mg) * c);
      }
      unsigned long long todo = __ballot(live);
      while (todo) {
        const int leader = __ffsll((long long)todo) - 1;
        const uint32_t kv = __shfl(v, leader, kWave);
        const bool member = live && v == kv;
        const Real sum = wave_sum_fixed<Real>(member ? c : Real(0));
        if (lane == leader) ordered_add<Real, LDS_ACC>(accT + kv, sum);
        todo &= ~__ballot(member);
      }
      __syncthreads();
    }
  }

  if (LDS_ACC) {
    __syncthreads();
    if (dw)
      for (long long i = lane; i < nW; i += kWave) dw[(long long)t * nW + i] = accW[i];
    if (dthr)
      for (int i = lane; i < d.V; i += kWave) dthr[(long long)t * d.V + i] = accT[i];
  }
}

template <typename Real, bool FERN>
int backward_deterministic(const ForestDims &d, const Real *x, const Real *thr, const int64_t *ord, const Real *w,
                           const Real *gout, Real *dx, Real *dthr, Real *dw, void *ws, size_t ws_bytes,
                           hipStream_t stream) {
  if (ws_bytes < records_bytes<Real>(d) || ws == nullptr)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: workspace too small for the deterministic backward pass.");
  Records<Real> rec = carve_records<Real>(d, ws);
  int rc = dispatch_records<Real, FERN>(d, x, thr, ord, rec, stream);
  if (rc != HT_OK) return rc;
  if (dx) {
    const long long blocks = (d.S + 255) / 256;
    hipLaunchKernelGGL(det_dx_kernel<Real>, dim3((unsigned)blocks), dim3(256), 0, stream, d, ord, w, gout, rec, dx);
    HT_LAUNCH_CHECK("deterministic dX");
  }
  if (dthr || dw) {
    const size_t need = (dw ? size_t(d.L) * d.M : 0) * sizeof(Real) + (dthr ? size_t(d.V) : 0) * sizeof(Real);
    if (need <= size_t(kLdsBytes) / 3) {
      auto kernel = det_tree_kernel<Real, true>;
      HT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, int(need)));
      hipLaunchKernelGGL(kernel, dim3((unsigned)d.T), dim3(kWave), need, stream, d, w, gout, rec, dthr, dw);
    } else {
      hipLaunchKernelGGL((det_tree_kernel<Real, false>), dim3((unsigned)d.T), dim3(kWave), 0, stream, d, w, gout, rec,
                         dthr, dw);
    }
    HT_LAUNCH_CHECK("deterministic dThr/dW");
  }
  return HT_OK;
}

}  // namespace

template <typename Real>
size_t forest_backward_workspace(const ForestDims &d, int mode) {
  return mode == HT_BACKWARD_DETERMINISTIC ? records_bytes<Real>(d) : 0;
}

template <typename Real>
int forest_backward(const ForestDims &d, bool fern, const Real *x, const Real *thr, const int64_t *ord, const Real *w,
                    const Real *gout, Real *dx, Real *dthr, Real *dw, int mode, void *ws, size_t ws_bytes,
                    hipStream_t stream) {
  int rc;
  if (dx && (rc = zero_fill(dx, size_t(d.S) * d.F * sizeof(Real), stream)) != HT_OK) return rc;
  if (dthr && (rc = zero_fill(dthr, size_t(d.T) * d.V * sizeof(Real), stream)) != HT_OK) return rc;
  if (dw && (rc = zero_fill(dw, size_t(d.T) * d.L * d.M * sizeof(Real), stream)) != HT_OK) return rc;
  if (d.S == 0 || d.T == 0 || (!dx && !dthr && !dw)) return HT_OK;
  if (mode == HT_BACKWARD_DETERMINISTIC)
    return fern ? backward_deterministic<Real, true>(d, x, thr, ord, w, gout, dx, dthr, dw, ws, ws_bytes, stream)
                : backward_deterministic<Real, false>(d, x, thr, ord, w, gout, dx, dthr, dw, ws, ws_bytes, stream);
  return fern ? dispatch_backward_atomic<Real, true>(d, x, thr, ord, w, gout, dx, dthr, dw, stream)
              : dispatch_backward_atomic<Real, false>(d, x, thr, ord, w, gout, dx, dthr, dw, stream);
}

template size_t forest_backward_workspace<float>(const ForestDims &, int);
template size_t forest_backward_workspace<double>(const ForestDims &, int);
template int forest_backward<float>(const ForestDims &, bool, const float *, const float *, const int64_t *,
                                    const float *, const float *, float *, float *, float *, int, void *, size_t,
                                    hipStream_t);
template int forest_backward<double>(const ForestDims &, bool, const double *, const double *, const int64_t *,
                                     const double *, const double *, double *, double *, double *, int, void *, size_t,
                                     hipStream_t);

}  // namespace ht
