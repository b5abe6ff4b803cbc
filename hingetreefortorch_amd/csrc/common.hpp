// Shared host/device helpers of libhingetree_hip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string>

#include "../../include/hingetree_hip.h"

namespace ht {

// ---- error reporting ------------------------------------------------------------------------------------------
void set_error(const std::string &msg);
int fail(int code, const std::string &msg);

#define HT_HIP_CHECK(expr)                                                                             \
  do {                                                                                                 \
    hipError_t ht_e_ = (expr);                                                                         \
    if (ht_e_ != hipSuccess)                                                                           \
      return ::ht::fail(HT_ERR_HIP, std::string(#expr) + " failed: " + hipGetErrorString(ht_e_));      \
  } while (0)

#define HT_LAUNCH_CHECK(what)                                                                          \
  do {                                                                                                 \
    hipError_t ht_e_ = hipGetLastError();                                                              \
    if (ht_e_ != hipSuccess)                                                                           \
      return ::ht::fail(HT_ERR_HIP, std::string("launch of ") + what + " failed: " + hipGetErrorString(ht_e_)); \
  } while (0)

// ---- shapes ----------------------------------------------------------------------------------------------------
// Sizes as the kernels see them. S = B*K is the number of independent "samples" (one per batch row and inner-data
// position); sample s lives at x[(s / K) * F * K + f * K + (s % K)].
struct ForestDims {
  long long S;   // B * K
  long long FK;  // F * K
  int F, K, T, depth, V, L, M;
};

__host__ __device__ constexpr size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

constexpr int kWave = 64;
constexpr int kLdsBytes = 160 * 1024;       // LDS per CU / per workgroup limit on gfx950
constexpr int kForestThreads = 1024;        // workgroup size of the tile kernels

// Validates a forest shape and derives ForestDims. Returns HT_OK or an error (message set).
int make_dims(const ht_forest_shape *s, ForestDims *d);

// ---- entry points implemented per translation unit -------------------------------------------------------------
template <typename Real>
int forest_forward(const ForestDims &d, bool fern, const Real *x, const Real *thr, const int64_t *ord, const Real *w,
                   Real *out, hipStream_t stream);

template <typename Real>
size_t forest_backward_workspace(const ForestDims &d, int mode);
template <typename Real>
int forest_backward(const ForestDims &d, bool fern, const Real *x, const Real *thr, const int64_t *ord, const Real *w,
                    const Real *gout, Real *dx, Real *dthr, Real *dw, int mode, void *ws, size_t ws_bytes,
                    hipStream_t stream);

template <typename Real>
int forest_maps(const ForestDims &d, bool fern, const Real *x, const Real *thr, const int64_t *ord, int64_t *leafmap,
                Real *margins, int64_t *ordinals, int64_t *reach, hipStream_t stream);

template <typename Real>
int conv_forward(const ht_conv_shape &s, const Real *x, const Real *thr, const int64_t *ord, const Real *w, Real *out,
                 hipStream_t stream);
template <typename Real>
int conv_backward(const ht_conv_shape &s, const Real *x, const Real *thr, const int64_t *ord, const Real *w,
                  const Real *gout, Real *dx, Real *dthr, Real *dw, hipStream_t stream);

int conv_output_size(const ht_conv_shape &s, int64_t *out_size);
int ordinal_range(const int64_t *ord, int64_t n, int64_t *minmax, hipStream_t stream);

// Fills n elements with zero through a kernel (safe to record into a HIP graph, unlike a memset node).
int zero_fill(void *p, size_t bytes, hipStream_t stream);

}  // namespace ht
