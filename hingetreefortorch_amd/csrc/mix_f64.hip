// Linear mix over the tree axis behind a forest, float64 (the reference's fused-linear operators instantiated for
// double, hingetree_fused_linear.cpp:798-806,845-853): plain kernels on the vector units. float64 is the precision
// of gradient checks and small problems; the matrix-core path in projection.hip serves float32.
//   forward : out[b, o, r] = bias[o] + sum_t lin[o, t] * f[b, t, r]
//   backward: h[b, t, r]   = sum_o lin[o, t] * g[b, o, r]
//             dlin[o, t]   = sum_{b, r} g[b, o, r] * f[b, t, r]
// Every sum runs in a fixed order, so all three results are reproducible run to run.
#include <hip/hip_runtime.h>

#include "common.hpp"

namespace ht {
namespace {

constexpr int kMixThreads = 256;

// c[b, i, r] = bias[i] + sum_j a(i, j) * v[b, j, r], with a(i, j) = A[i * lda_i + j * lda_j]; one thread per (b, i, r),
// r fastest (consecutive threads read consecutive r of v).
__global__ __launch_bounds__(kMixThreads) void mix_apply_kernel(const double *__restrict__ A, long long lda_i,
                                                                long long lda_j, const double *__restrict__ v,
                                                                const double *__restrict__ bias, double *__restrict__ c,
                                                                long long B, long long NI, long long NJ, long long R) {
  const long long total = B * NI * R;
  for (long long at = (long long)blockIdx.x * kMixThreads + threadIdx.x; at < total;
       at += (long long)gridDim.x * kMixThreads) {
    const long long r = at % R, bi = at / R;
    const long long i = bi % NI, b = bi / NI;
    double sum = bias ? bias[i] : 0.0;
    const double *row = A + i * lda_i;
    const double *col = v + b * NJ * R + r;
    for (long long j = 0; j < NJ; ++j) sum += row[j * lda_j] * col[j * R];
    c[at] = sum;
  }
}

// dlin[o, t] = sum_{b, r} g[b, o, r] * f[b, t, r]: one workgroup per (o, t); each thread sums a strided share of the
// (b, r) pairs in ascending order, and the shares meet in a fixed tree in LDS.
__global__ __launch_bounds__(kMixThreads) void mix_dlin_kernel(const double *__restrict__ g, const double *__restrict__ f,
                                                               double *__restrict__ dlin, long long B, long long T,
                                                               long long O, long long R) {
  __shared__ double part[kMixThreads];
  for (long long cell = blockIdx.x; cell < O * T; cell += gridDim.x) {
    const long long o = cell / T, t = cell % T;
    double sum = 0.0;
    for (long long p = threadIdx.x; p < B * R; p += kMixThreads) {
      const long long b = p / R, r = p - b * R;
      sum += g[(b * O + o) * R + r] * f[(b * T + t) * R + r];
    }
    part[threadIdx.x] = sum;
    __syncthreads();
    for (int half = kMixThreads / 2; half > 0; half >>= 1) {
      if (int(threadIdx.x) < half) part[threadIdx.x] += part[threadIdx.x + half];
      __syncthreads();
    }
    if (threadIdx.x == 0) dlin[cell] = part[0];
    __syncthreads();
  }
}

unsigned grid_for(long long items, long long per_block) {
  long long blocks = (items + per_block - 1) / per_block;
  const long long cap = 64ll * kNumCUs;
  if (blocks > cap) blocks = cap;
  return unsigned(blocks < 1 ? 1 : blocks);
}

}  // namespace

int mix_forward_f64(long long B, long long T, long long O, long long R, const double *f, const double *lin,
                    const double *bias, double *out, hipStream_t stream) {
  if (B * O * R == 0) return HT_OK;
  hipLaunchKernelGGL(mix_apply_kernel, dim3(grid_for(B * O * R, kMixThreads)), dim3(kMixThreads), 0, stream, lin, T, 1ll,
                     f, bias, out, B, O, T, R);
  HT_LAUNCH_CHECK("linear mix (float64)");
  return HT_OK;
}

int mix_backward_f64(long long B, long long T, long long O, long long R, const double *f, const double *lin,
                     const double *g, double *h, double *dlin, hipStream_t stream) {
  if (h && B * T * R != 0) {
    // h[b, t, r] = sum_o lin[o, t] * g[b, o, r]: the matrix is read transposed
    hipLaunchKernelGGL(mix_apply_kernel, dim3(grid_for(B * T * R, kMixThreads)), dim3(kMixThreads), 0, stream, lin, 1ll,
                       T, g, (const double *)nullptr, h, B, T, O, R);
    HT_LAUNCH_CHECK("linear mix backward (float64)");
  }
  if (dlin && O * T != 0) {
    hipLaunchKernelGGL(mix_dlin_kernel, dim3(grid_for(O * T, 1)), dim3(kMixThreads), 0, stream, g, f, dlin, B, T, O, R);
    HT_LAUNCH_CHECK("linear mix weight gradient (float64)");
  }
  return HT_OK;
}

}  // namespace ht
