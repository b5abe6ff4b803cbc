// Forest / fern forward: out[b,t,k,m] = |margin| * w[t,leaf,m].
//
// One workgroup = one tile of BT samples (all features in LDS, feature major) x a range of trees. Per pass the
// NT/BT tree slots walk one tree each (lane = sample), park (|margin|, leaf) in LDS, and then the whole workgroup
// writes the pass' outputs with the thread index running along the contiguous (tree, m) -- or for K > 1 the
// contiguous (inner position, m) -- axis of `out`, so the dominant store traffic is emitted as full-width rows.
#include "forest_tile.hpp"

namespace ht {
namespace {

template <typename Real, bool FERN, int BT, bool XLDS>
__global__ __launch_bounds__(kForestThreads) void forward_kernel(ForestDims d, const Real *__restrict__ x,
                                                                 const Real *__restrict__ thr,
                                                                 const int64_t *__restrict__ ord,
                                                                 const Real *__restrict__ w, Real *__restrict__ out,
                                                                 int trees_per_block) {
  constexpr int NT = kForestThreads;
  constexpr int TC = NT / BT;  // trees walked per pass
  extern __shared__ __align__(16) unsigned char smem[];
  Real *xs = reinterpret_cast<Real *>(smem);
  Real *r_abs = xs + (XLDS ? size_t(d.F) * BT : 0);
  uint32_t *r_key = reinterpret_cast<uint32_t *>(r_abs + TC * BT);

  const long long s0 = (long long)blockIdx.x * BT;
  if (XLDS) {
    load_tile<Real, BT, NT>(xs, x, d, s0);
    __syncthreads();
  }
  const int j = threadIdx.x % BT, tt = threadIdx.x / BT;
  const long long s = s0 + j;
  const bool live = s < d.S;
  const long long xbase = live ? (s / d.K) * d.FK + (s % d.K) : 0;

  const int t_begin = blockIdx.y * trees_per_block;
  const int t_end = min(d.T, t_begin + trees_per_block);
  for (int tb = t_begin; tb < t_end; tb += TC) {
    const int t = tb + tt;
    if (t < t_end && live) {
      const Real *th = thr + (long long)t * d.V;
      const int64_t *od = ord + (long long)t * d.V;
      auto node = [&](uint32_t at, Real &tv, int &ov) { tv = th[at]; ov = clamp_ordinal(od[at], d.F); };
      WalkResult<Real> r;
      if (XLDS)
        r = walk<Real, FERN>(d.depth, node, [&](int f) { return xs[f * BT + j]; });
      else
        r = walk<Real, FERN>(d.depth, node, [&](int f) { return x[xbase + (long long)f * d.K]; });
      r_abs[tt * BT + j] = ht_abs(r.margin);
      r_key[tt * BT + j] = r.key;
    }
    __syncthreads();
    const int nt = min(TC, t_end - tb);
    if (d.K == 1) {
      // out[s, tb .. tb+nt, 0 .. M) is contiguous for a fixed sample
      const int row = nt * d.M, total = BT * row;
      for (int idx = threadIdx.x; idx < total; idx += NT) {
        const int jj = idx / row, r = idx - jj * row;
        const int t2 = r / d.M, m = r - t2 * d.M;
        const long long ss = s0 + jj;
        if (ss < d.S) {
          const uint32_t key = r_key[t2 * BT + jj];
          out[(ss * d.T + tb) * d.M + r] = r_abs[t2 * BT + jj] * w[((long long)(tb + t2) * d.L + key) * d.M + m];
        }
      }
    } else {
      // out[b, t, k .. , 0 .. M) is contiguous for a fixed tree
      const int row = BT * d.M, total = nt * row;
      for (int idx = threadIdx.x; idx < total; idx += NT) {
        const int t2 = idx / row, r = idx - t2 * row;
        const int jj = r / d.M, m = r - jj * d.M;
        const long long ss = s0 + jj;
        if (ss < d.S) {
          const uint32_t key = r_key[t2 * BT + jj];
          out[out_offset(d, ss, tb + t2, m)] = r_abs[t2 * BT + jj] * w[((long long)(tb + t2) * d.L + key) * d.M + m];
        }
      }
    }
    __syncthreads();
  }
}

template <typename Real, bool FERN, int BT, bool XLDS>
int launch_forward(const ForestDims &d, const Real *x, const Real *thr, const int64_t *ord, const Real *w, Real *out,
                   hipStream_t stream) {
  constexpr int TC = kForestThreads / BT;
  const size_t lds = (XLDS ? size_t(d.F) * BT * sizeof(Real) : 0) + size_t(TC) * BT * (sizeof(Real) + sizeof(uint32_t));
  const long long tiles = (d.S + BT - 1) / BT;
  // Split the trees over blockIdx.y when there are too few sample tiles to fill 256 CUs.
  const int passes = (d.T + TC - 1) / TC;
  long long want = tiles >= 512 ? 1 : (512 + tiles - 1) / tiles;
  const int split = int(want < passes ? want : passes);
  const int trees_per_block = ((passes + split - 1) / split) * TC;
  const int gy = (d.T + trees_per_block - 1) / trees_per_block;
  if (tiles > 0x7fffffffLL) return fail(HT_ERR_RUNTIME, "Error: too many sample tiles for one launch.");
  auto kernel = forward_kernel<Real, FERN, BT, XLDS>;
  HT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   int(lds)));
  hipLaunchKernelGGL(kernel, dim3((unsigned)tiles, (unsigned)gy), dim3(kForestThreads), lds, stream, d, x, thr, ord, w,
                     out, trees_per_block);
  HT_LAUNCH_CHECK("forest forward");
  return HT_OK;
}

template <typename Real, bool FERN>
int dispatch_forward(const ForestDims &d, const Real *x, const Real *thr, const int64_t *ord, const Real *w, Real *out,
                     hipStream_t stream) {
  const size_t reserve = 16 * 1024;
  switch (pick_tile<Real>(d.F, reserve)) {
    case 64: return launch_forward<Real, FERN, 64, true>(d, x, thr, ord, w, out, stream);
    case 32: return launch_forward<Real, FERN, 32, true>(d, x, thr, ord, w, out, stream);
    case 16: return launch_forward<Real, FERN, 16, true>(d, x, thr, ord, w, out, stream);
    case 8: return launch_forward<Real, FERN, 8, true>(d, x, thr, ord, w, out, stream);
    default: return launch_forward<Real, FERN, 64, false>(d, x, thr, ord, w, out, stream);
  }
}

}  // namespace

template <typename Real>
int forest_forward(const ForestDims &d, bool fern, const Real *x, const Real *thr, const int64_t *ord, const Real *w,
                   Real *out, hipStream_t stream) {
  if (d.S == 0 || d.T == 0) return HT_OK;
  return fern ? dispatch_forward<Real, true>(d, x, thr, ord, w, out, stream)
              : dispatch_forward<Real, false>(d, x, thr, ord, w, out, stream);
}

template int forest_forward<float>(const ForestDims &, bool, const float *, const float *, const int64_t *, const float *,
                                   float *, hipStream_t);
template int forest_forward<double>(const ForestDims &, bool, const double *, const double *, const int64_t *,
                                    const double *, double *, hipStream_t);

}  // namespace ht
