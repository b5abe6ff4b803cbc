// Convolutional hinge trees / ferns (1, 2 or 3 spatial dims, groups == 1).
//
// out[b, j, p, m] = sum_c |margin_{j,c}(patch_c(p))| * w[j, c, leaf, m]: one tree per (out channel j, in channel c)
// over the P = prod(kernel) taps of channel c's patch around output position p. The reference materialises the
// patches (im2col) per (image, channel); here a tap index is turned into an image coordinate inside the walk, taps
// in the padding read 0, and nothing but x, the parameters and out touches memory.
//
// Forward accumulates over c in ascending order from +0 with separate multiply and add (the translation unit is
// built with -ffp-contract=off), which reproduces the reference's `out += w * |margin|` bit for bit.
#include "common.hpp"
#include "walk.hpp"

namespace ht {
namespace {

struct ConvGeom {
  int nd;
  int size[3], osz[3], ker[3], str[3], pad[3], dil[3];
  int rows;      // output positions per (image, channel)
  int taps;      // P
  int in_count;  // input positions per (image, channel)
};

constexpr int kConvThreads = 256;
constexpr int kMaxRegM = 16;

// Offsets of tap j relative to the patch anchor, per dim (already multiplied by the dilation): tapc[j * 3 + d].
__device__ __forceinline__ void fill_tap_table(int *tapc, const ConvGeom &g) {
  for (int j = threadIdx.x; j < g.taps; j += blockDim.x) {
    int rest = j;
    int c[3] = {0, 0, 0};
    for (int dd = g.nd - 1; dd >= 0; --dd) {
      c[dd] = (rest % g.ker[dd]) * g.dil[dd];
      rest /= g.ker[dd];
    }
    tapc[j * 3 + 0] = c[0];
    tapc[j * 3 + 1] = c[1];
    tapc[j * 3 + 2] = c[2];
  }
}

// Flat offset inside one channel image of tap `tap` for the patch anchored at `anchor`, or -1 in the padding.
__device__ __forceinline__ int tap_offset(const ConvGeom &g, const int *tapc, const int anchor[3], int tap) {
  int flat = 0;
  bool inside = true;
  for (int dd = 0; dd < g.nd; ++dd) {
    const int at = anchor[dd] + tapc[tap * 3 + dd];
    inside = inside && at >= 0 && at < g.size[dd];
    flat = flat * g.size[dd] + at;
  }
  return inside ? flat : -1;
}

__device__ __forceinline__ void anchor_of(const ConvGeom &g, int p, int anchor[3]) {
  int rest = p;
  anchor[0] = anchor[1] = anchor[2] = 0;
  for (int dd = g.nd - 1; dd >= 0; --dd) {
    anchor[dd] = (rest % g.osz[dd]) * g.str[dd] - g.pad[dd];
    rest /= g.osz[dd];
  }
}

template <typename Real, bool FERN>
__global__ __launch_bounds__(kConvThreads) void conv_forward_kernel(ConvGeom g, int C, int Cout, int depth, int V, int L,
                                                                    int M, const Real *__restrict__ x,
                                                                    const Real *__restrict__ thr,
                                                                    const int64_t *__restrict__ ord,
                                                                    const Real *__restrict__ w, Real *__restrict__ out) {
  extern __shared__ __align__(16) unsigned char smem[];
  int *tapc = reinterpret_cast<int *>(smem);
  fill_tap_table(tapc, g);
  __syncthreads();
  const int p = blockIdx.x * kConvThreads + threadIdx.x;
  const int j = blockIdx.y;
  const long long b = blockIdx.z;
  if (p >= g.rows) return;
  int anchor[3];
  anchor_of(g, p, anchor);
  Real *o = out + ((b * Cout + j) * (long long)g.rows + p) * M;
  for (int m0 = 0; m0 < M; m0 += kMaxRegM) {
    const int mc = min(kMaxRegM, M - m0);
    Real acc[kMaxRegM];
#pragma unroll
    for (int m = 0; m < kMaxRegM; ++m) acc[m] = Real(0);
    for (int c = 0; c < C; ++c) {
      const Real *img = x + (b * C + c) * (long long)g.in_count;
      const long long tree = (long long)j * C + c;
      const Real *th = thr + tree * V;
      const int64_t *od = ord + tree * V;
      const WalkResult<Real> r = walk<Real, FERN>(
          depth, [&](uint32_t at, Real &tv, int &ov) { tv = th[at]; ov = clamp_ordinal(od[at], g.taps); },
          [&](int tap) {
            const int off = tap_offset(g, tapc, anchor, tap);
            return off < 0 ? Real(0) : img[off];
          });
      const Real a = ht_abs(r.margin);
      const Real *wl = w + (tree * L + r.key) * M + m0;
#pragma unroll
      for (int m = 0; m < kMaxRegM; ++m)
        if (m < mc) acc[m] = acc[m] + wl[m] * a;
    }
#pragma unroll
    for (int m = 0; m < kMaxRegM; ++m)
      if (m < mc) o[m0 + m] = acc[m];
  }
}

// Backward. LDS_ACC: dThr[j,c,:] and dW[j,c,:,:] of the block's (j, c) tree are accumulated in LDS over the block's
// 256 positions and flushed with one global atomic per touched cell.
template <typename Real, bool FERN, bool LDS_ACC>
__global__ __launch_bounds__(kConvThreads) void conv_backward_kernel(ConvGeom g, int C, int Cout, int depth, int V,
                                                                     int L, int M, const Real *__restrict__ x,
                                                                     const Real *__restrict__ thr,
                                                                     const int64_t *__restrict__ ord,
                                                                     const Real *__restrict__ w,
                                                                     const Real *__restrict__ gout, Real *dx,
                                                                     Real *dthr, Real *dw) {
  extern __shared__ __align__(16) unsigned char smem[];
  int *tapc = reinterpret_cast<int *>(smem);
  Real *accT = reinterpret_cast<Real *>(smem + align_up(size_t(g.taps) * 3 * sizeof(int), 16));
  Real *accW = accT + V;
  fill_tap_table(tapc, g);
  __syncthreads();
  const int p = blockIdx.x * kConvThreads + threadIdx.x;
  const int j = blockIdx.y;
  const long long b = blockIdx.z;
  const bool live = p < g.rows;
  int anchor[3] = {0, 0, 0};
  if (live) anchor_of(g, p, anchor);
  const Real *gp = gout + ((b * Cout + j) * (long long)g.rows + (live ? p : 0)) * M;
  const int nacc = V + L * M;
  for (int c = 0; c < C; ++c) {
    const long long tree = (long long)j * C + c;
    if (LDS_ACC) {
      for (int i = threadIdx.x; i < nacc; i += kConvThreads) accT[i] = Real(0);
      __syncthreads();
    }
    if (live) {
      const Real *img = x + (b * C + c) * (long long)g.in_count;
      const Real *th = thr + tree * V;
      const int64_t *od = ord + tree * V;
      const WalkResult<Real> r = walk<Real, FERN>(
          depth, [&](uint32_t at, Real &tv, int &ov) { tv = th[at]; ov = clamp_ordinal(od[at], g.taps); },
          [&](int tap) {
            const int off = tap_offset(g, tapc, anchor, tap);
            return off < 0 ? Real(0) : img[off];
          });
      const Real a = ht_abs(r.margin);
      const Real *wl = w + (tree * L + r.key) * M;
      Real cs = Real(0);
      for (int m = 0; m < M; ++m) {
        const Real gv = gp[m];
        cs += wl[m] * gv;
        if (dw) {
          if (LDS_ACC)
            atomicAdd(accW + (long long)r.key * M + m, a * gv);
          else
            atomicAdd(dw + (tree * L + r.key) * M + m, a * gv);
        }
      }
      cs = ht_sign(r.margin) * cs;
      if (dthr) {
        if (LDS_ACC)
          atomicAdd(accT + r.vertex, -cs);
        else
          atomicAdd(dthr + tree * V + r.vertex, -cs);
      }
      if (dx) {
        const int off = tap_offset(g, tapc, anchor, int(od[r.vertex]));
        if (off >= 0) atomicAdd(dx + (b * C + c) * (long long)g.in_count + off, cs);
      }
    }
    if (LDS_ACC) {
      __syncthreads();
      if (dthr)
        for (int i = threadIdx.x; i < V; i += kConvThreads)
          if (accT[i] != Real(0)) atomicAdd(dthr + tree * V + i, accT[i]);
      if (dw)
        for (int i = threadIdx.x; i < L * M; i += kConvThreads)
          if (accW[i] != Real(0)) atomicAdd(dw + tree * L * M + i, accW[i]);
      __syncthreads();
    }
  }
}

int make_geom(const ht_conv_shape &s, ConvGeom *g) {
  if (s.nd < 1 || s.nd > HT_MAX_CONV_DIMS)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: convolution supports 1, 2 or 3 spatial dimensions.");
  long long rows = 1, taps = 1, in_count = 1;
  g->nd = s.nd;
  for (int d = 0; d < 3; ++d) {
    g->size[d] = g->osz[d] = g->ker[d] = g->str[d] = g->dil[d] = 1;
    g->pad[d] = 0;
  }
  for (int d = 0; d < s.nd; ++d) {
    // validity rules of ImageToMatrix.h:159-183
    if (s.kernel[d] <= 0 || s.stride[d] <= 0 || s.dilation[d] <= 0 || s.padding[d] < 0 || s.size[d] < 1)
      return fail(HT_ERR_RUNTIME, "Error: Unable to convert image patches to matrix.");
    const long long win = s.kernel[d] + (s.kernel[d] - 1) * (s.dilation[d] - 1);
    if (s.size[d] + 2 * s.padding[d] < win)
      return fail(HT_ERR_RUNTIME, "Error: Unable to convert image patches to matrix.");
    const long long osz = (s.size[d] + 2 * s.padding[d] - win) / s.stride[d] + 1;  // ImageToMatrix.h:201-209
    g->size[d] = int(s.size[d]);
    g->osz[d] = int(osz);
    g->ker[d] = int(s.kernel[d]);
    g->str[d] = int(s.stride[d]);
    g->pad[d] = int(s.padding[d]);
    g->dil[d] = int(s.dilation[d]);
    rows *= osz;
    taps *= s.kernel[d];
    in_count *= s.size[d];
  }
  if (rows > 0x7fffffffLL || in_count > 0x7fffffffLL || taps > 4096)
    return fail(HT_ERR_RUNTIME, "Error: convolution geometry too large for this build.");
  if (s.B > 65535 || s.Cout > 65535)
    return fail(HT_ERR_RUNTIME, "Error: batch size and out channels are limited to 65535 in the convolution kernels.");
  g->rows = int(rows);
  g->taps = int(taps);
  g->in_count = int(in_count);
  return HT_OK;
}

}  // namespace

int conv_output_size(const ht_conv_shape &s, int64_t *out_size) {
  ConvGeom g;
  int rc = make_geom(s, &g);
  if (rc != HT_OK) return rc;
  for (int d = 0; d < s.nd; ++d) out_size[d] = g.osz[d];
  return HT_OK;
}

template <typename Real>
int conv_forward(const ht_conv_shape &s, const Real *x, const Real *thr, const int64_t *ord, const Real *w, Real *out,
                 hipStream_t stream) {
  ConvGeom g;
  int rc = make_geom(s, &g);
  if (rc != HT_OK) return rc;
  if (s.B == 0 || s.Cout == 0 || g.rows == 0) return HT_OK;
  const bool fern = s.kind == HT_FERN;
  const int V = fern ? int(s.depth) : int((1LL << s.depth) - 1), L = int(1LL << s.depth);
  if (s.C == 0) return zero_fill(out, size_t(s.B) * s.Cout * g.rows * s.M * sizeof(Real), stream);
  const dim3 grid((g.rows + kConvThreads - 1) / kConvThreads, (unsigned)s.Cout, (unsigned)s.B);
  const size_t lds = size_t(g.taps) * 3 * sizeof(int);
  if (fern)
    hipLaunchKernelGGL((conv_forward_kernel<Real, true>), grid, dim3(kConvThreads), lds, stream, g, int(s.C),
                       int(s.Cout), int(s.depth), V, L, int(s.M), x, thr, ord, w, out);
  else
    hipLaunchKernelGGL((conv_forward_kernel<Real, false>), grid, dim3(kConvThreads), lds, stream, g, int(s.C),
                       int(s.Cout), int(s.depth), V, L, int(s.M), x, thr, ord, w, out);
  HT_LAUNCH_CHECK("conv forward");
  return HT_OK;
}

template <typename Real, bool FERN, bool LDS_ACC>
int launch_conv_backward(const ConvGeom &g, const ht_conv_shape &s, int V, int L, size_t lds, const Real *x,
                         const Real *thr, const int64_t *ord, const Real *w, const Real *gout, Real *dx, Real *dthr,
                         Real *dw, hipStream_t stream) {
  const dim3 grid((g.rows + kConvThreads - 1) / kConvThreads, (unsigned)s.Cout, (unsigned)s.B);
  auto kernel = conv_backward_kernel<Real, FERN, LDS_ACC>;
  HT_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   int(lds)));
  hipLaunchKernelGGL(kernel, grid, dim3(kConvThreads), lds, stream, g, int(s.C), int(s.Cout), int(s.depth), V, L,
                     int(s.M), x, thr, ord, w, gout, dx, dthr, dw);
  HT_LAUNCH_CHECK("conv backward");
  return HT_OK;
}

template <typename Real>
int conv_backward(const ht_conv_shape &s, const Real *x, const Real *thr, const int64_t *ord, const Real *w,
                  const Real *gout, Real *dx, Real *dthr, Real *dw, hipStream_t stream) {
  ConvGeom g;
  int rc = make_geom(s, &g);
  if (rc != HT_OK) return rc;
  const bool fern = s.kind == HT_FERN;
  const int V = fern ? int(s.depth) : int((1LL << s.depth) - 1), L = int(1LL << s.depth);
  if (dx && (rc = zero_fill(dx, size_t(s.B) * s.C * g.in_count * sizeof(Real), stream)) != HT_OK) return rc;
  if (dthr && (rc = zero_fill(dthr, size_t(s.Cout) * s.C * V * sizeof(Real), stream)) != HT_OK) return rc;
  if (dw && (rc = zero_fill(dw, size_t(s.Cout) * s.C * L * s.M * sizeof(Real), stream)) != HT_OK) return rc;
  if (s.B == 0 || s.Cout == 0 || s.C == 0 || g.rows == 0 || (!dx && !dthr && !dw)) return HT_OK;
  const size_t tap_bytes = align_up(size_t(g.taps) * 3 * sizeof(int), 16);
  const size_t acc_bytes = (size_t(V) + size_t(L) * s.M) * sizeof(Real);
  const bool lds_acc = acc_bytes <= 48 * 1024;
  const size_t lds = tap_bytes + (lds_acc ? acc_bytes : 0);
  if (fern)
    return lds_acc ? launch_conv_backward<Real, true, true>(g, s, V, L, lds, x, thr, ord, w, gout, dx, dthr, dw, stream)
                   : launch_conv_backward<Real, true, false>(g, s, V, L, lds, x, thr, ord, w, gout, dx, dthr, dw, stream);
  return lds_acc ? launch_conv_backward<Real, false, true>(g, s, V, L, lds, x, thr, ord, w, gout, dx, dthr, dw, stream)
                 : launch_conv_backward<Real, false, false>(g, s, V, L, lds, x, thr, ord, w, gout, dx, dthr, dw, stream);
}

template int conv_forward<float>(const ht_conv_shape &, const float *, const float *, const int64_t *, const float *,
                                 float *, hipStream_t);
template int conv_forward<double>(const ht_conv_shape &, const double *, const double *, const int64_t *, const double *,
                                  double *, hipStream_t);
template int conv_backward<float>(const ht_conv_shape &, const float *, const float *, const int64_t *, const float *,
                                  const float *, float *, float *, float *, hipStream_t);
template int conv_backward<double>(const ht_conv_shape &, const double *, const double *, const int64_t *,
                                   const double *, const double *, double *, double *, double *, hipStream_t);

}  // namespace ht
