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

// No (sample, tree, output) triple exists: outputs are empty and every gradient is zero.
inline bool is_empty(const ForestDims &d) { return d.S == 0 || d.T == 0 || d.M == 0; }

__host__ __device__ constexpr size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

constexpr int kWave = 64;
constexpr int kLdsBytes = 160 * 1024;       // LDS per CU / per workgroup limit on gfx950
constexpr int kForestThreads = 1024;        // workgroup size of the tile kernels
constexpr int kNumCUs = 256;                // MI355X
constexpr int kNumXCDs = 8;                 // accelerator dies, each with its own L2; workgroup i runs on XCD i mod 8

// n / d for n * d < 2^32 by multiply-high with ceil(2^32 / d) (d >= 1).
struct FastDiv {
  uint32_t inv;
  uint32_t d;
  __host__ __device__ FastDiv() : inv(0), d(1) {}
  __host__ __device__ explicit FastDiv(int divisor) : inv(divisor <= 1 ? 0u : uint32_t(((1ull << 32) + divisor - 1) / divisor)), d(divisor) {}
  __device__ __forceinline__ int div(int n) const { return d <= 1 ? n : int(__umulhi(uint32_t(n), inv)); }
};

// Where a forest with inner data positions [tiles...] and outputs per leaf [window...] stores its result when the caller
// wants the image that the expand permutation would make of it: element (position k, output m) of a (sample, tree)
// plane goes to image coordinate tile * window + within - padding of every dimension, and is dropped outside the image.
// Dimensions are right-aligned in the arrays (a 2-d geometry has a leading dimension of extent 1). nd == 0: off.
struct ImageStore {
  int nd;
  int tiles[3], win[3], pad[3], size[3];
  FastDiv by_tiles[3], by_win[3];
  long long plane;  // elements of one (sample, tree) image
  __device__ __forceinline__ long long offset(int k, int m) const {
    int q = by_tiles[2].div(k);
    const int j2 = k - q * tiles[2];
    const int j0 = by_tiles[1].div(q), j1 = q - j0 * tiles[1];
    q = by_win[2].div(m);
    const int w2 = m - q * win[2];
    const int w0 = by_win[1].div(q), w1 = q - w0 * win[1];
    const int p0 = j0 * win[0] + w0 - pad[0], p1 = j1 * win[1] + w1 - pad[1], p2 = j2 * win[2] + w2 - pad[2];
    if (p0 < 0 || p0 >= size[0] || p1 < 0 || p1 >= size[1] || p2 < 0 || p2 >= size[2]) return -1;
    return ((long long)p0 * size[1] + p1) * size[2] + p2;
  }
};
// Validates the geometry against the forest's shape; *clear is set when the image has positions no tile covers.
int make_image_store(const ht_tile_shape *g, const ForestDims &d, long long B, ImageStore *img, bool *clear);

// How a tile kernel spreads the trees over blockIdx.y: with few sample tiles the trees are split so that at least
// ~2 workgroups per CU exist; `group` is the number of trees a workgroup handles per pass.
static inline void split_trees(long long tiles, int T, int group, int *trees_per_block, int *grid_y) {
  const int passes = (T + group - 1) / group;
  const long long want = tiles >= 2 * kNumCUs ? 1 : (2 * kNumCUs + tiles - 1) / (tiles > 0 ? tiles : 1);
  const int split = int(want < passes ? want : passes);
  *trees_per_block = ((passes + split - 1) / (split > 0 ? split : 1)) * group;
  *grid_y = (T + *trees_per_block - 1) / *trees_per_block;
}

// Validates a forest shape and derives ForestDims. Returns HT_OK or an error (message set).
int make_dims(const ht_forest_shape *s, ForestDims *d);

// ---- entry points implemented per translation unit -------------------------------------------------------------
// Packed (threshold, ordinal) vertices: layout in walk.hpp (Node<Real>), T*V entries.
template <typename Real>
size_t packed_nodes_bytes(const ForestDims &d);
// zero_slots (optional): kBoundSlots 64-bit words (records.hpp) that the same launch clears.
template <typename Real>
int pack_nodes(const ForestDims &d, const Real *thr, const int64_t *ord, void *dst, hipStream_t stream,
               unsigned long long *zero_slots = nullptr);

// Optional normalisation of the features on their way into the forward pass: feature f of every sample is read as
// (x - mean[f]) * rstd[f] (two rounded operations, like a separate elementwise pass would do them). Null: x as it is.
template <typename Real>
struct FeatureNorm {
  const Real *mean = nullptr, *rstd = nullptr;
};

template <typename Real>
size_t forest_forward_workspace(const ForestDims &d);
// `records` (optional): forest_records_bytes() bytes that receive the walk records for forest_backward_records().
// `image` (optional): store the result as that image instead of [B, T, K, M]; needs K > 1.
// `norm` (optional): the features are normalised as they are read (FeatureNorm).
template <typename Real>
int forest_forward(const ForestDims &d, bool fern, const Real *x, const Real *thr, const int64_t *ord, const Real *w,
                   Real *out, void *records, void *ws, size_t ws_bytes, hipStream_t stream,
                   const ImageStore *image = nullptr, const FeatureNorm<Real> *norm = nullptr);

template <typename Real>
size_t forest_backward_workspace(const ForestDims &d, int mode, bool need_dx, bool need_dthr, bool need_dw);
template <typename Real>
int forest_backward(const ForestDims &d, bool fern, const Real *x, const Real *thr, const int64_t *ord, const Real *w,
                    const Real *gout, Real *dx, Real *dthr, Real *dw, int mode, void *ws, size_t ws_bytes,
                    hipStream_t stream, const ImageStore *gout_image = nullptr);
// gout_image: gout is the image [B, T, *size] whose contraction by that tile geometry is the upstream gradient
// [B, T, *tiles, *window]; served where forest_backward_image_ok says so.
template <typename Real>
bool forest_backward_image_ok(const ForestDims &d, int mode, bool need_dx, bool need_dw, const ImageStore &img);

// Training path: backward from the records a forward pass wrote (0 bytes: not offered for this shape).
template <typename Real>
size_t forest_records_bytes(const ForestDims &d);
template <typename Real>
size_t forest_backward_records_workspace(const ForestDims &d, int mode, bool need_dx, bool need_dthr, bool need_dw);
template <typename Real>
int forest_backward_records(const ForestDims &d, bool fern, const Real *w, const Real *gout, const void *records,
                            Real *dx, Real *dthr, Real *dw, int mode, void *ws, size_t ws_bytes, hipStream_t stream);

// ... for dThr / dW alone, leaving c = sign(margin) * sum_m w * g of every pair, tree major [T][S], at the start of the
// workspace (*c) for a caller that goes on from the records itself; atomic mode, where forest_backward_keeps_c says so.
template <typename Real>
bool forest_backward_keeps_c(const ForestDims &d);
template <typename Real>
int forest_backward_records_keep_c(const ForestDims &d, bool fern, const Real *w, const Real *gout, const void *records,
                                   Real *dthr, Real *dw, void *ws, size_t ws_bytes, hipStream_t stream, const Real **c);

// The maps on the forward's row kernel walk (forest_forward.hip): bytes of packed vertices it wants (0: shape not
// served), and the launch; keys16 (optional) receives the leaf keys as 16-bit values tree major.
template <typename Real>
size_t forest_maps_rows_workspace(const ForestDims &d);
template <typename Real>
int forest_maps_rows(const ForestDims &d, bool fern, const Real *x, const Real *thr, const int64_t *ord,
                     int64_t *leafmap, uint16_t *keys16, Real *margins, int64_t *ordinals, void *ws, hipStream_t stream);

template <typename Real>
size_t forest_maps_workspace(const ForestDims &d, bool want_reach);
template <typename Real>
int forest_maps(const ForestDims &d, bool fern, const Real *x, const Real *thr, const int64_t *ord, int64_t *leafmap,
                Real *margins, int64_t *ordinals, int64_t *reach, void *ws, size_t ws_bytes, hipStream_t stream);

template <typename Real>
int conv_forward(const ht_conv_shape &s, const Real *x, const Real *thr, const int64_t *ord, const Real *w, Real *out,
                 hipStream_t stream);
template <typename Real>
int conv_backward(const ht_conv_shape &s, const Real *x, const Real *thr, const int64_t *ord, const Real *w,
                  const Real *gout, Real *dx, Real *dthr, Real *dw, hipStream_t stream);

int conv_output_size(const ht_conv_shape &s, int64_t *out_size);

// Linear mix over the tree axis behind a forest, float64 (mix_f64.hip; plain kernels, fixed summation order).
int mix_forward_f64(long long B, long long T, long long O, long long R, const double *f, const double *lin,
                    const double *bias, double *out, hipStream_t stream);
int mix_backward_f64(long long B, long long T, long long O, long long R, const double *f, const double *lin,
                     const double *g, double *h, double *dlin, hipStream_t stream);

// Linear mix over the tree axis behind a forest (projection.hip), fp32.
int rows_to_planes(long long n, long long R, const float *rows, float *planes, bool back, hipStream_t stream);
int mix_forward(long long B, long long T, long long O, long long R, const float *f, const float *lin,
                const float *bias, float *out, hipStream_t stream);
size_t mix_backward_workspace(long long B, long long T, long long O, long long R);
int mix_backward(long long B, long long T, long long O, long long R, const float *f, const float *lin, const float *g,
                 float *h, float *dlin, bool deterministic, hipStream_t stream, void *ws = nullptr, size_t ws_bytes = 0);

// Tile <-> image permutation (expand.hip).
int tile_contract(const ht_tile_shape *s, const void *in, void *out, hipStream_t stream);
int tile_expand(const ht_tile_shape *s, const void *in, void *out, hipStream_t stream);

// Dense projection + batch normalisation in front of a forest (projection.hip), fp32.
size_t projection_workspace(long long N);
size_t projection_backward_workspace(long long B, long long K, long long N);
int projection_forward(long long B, long long K, long long N, const float *x, const float *lin, double eps,
                       float *zhat, float *mean, float *rstd, float *var, void *ws, hipStream_t stream);
int projection_backward(long long B, long long K, long long N, const float *x, const float *lin, const float *zhat,
                        const float *rstd, float *g, float *dlin, float *dx, void *ws, hipStream_t stream);
// The same gradients for the whole Linear -> BatchNorm -> forest front from the forest's walk records: dThr, dW and
// dLin without a dense dL/dzhat (d: the forest over the N = d.F projected features of B = d.S samples, K_in inputs).
// (mean given: `zhat` is the un-normalised product z of projection_forest_forward)
bool projection_forest_backward_ok(const ForestDims &d, long long K_in);
// The forward pass of the front with the forest reading the un-normalised product z through FeatureNorm.
size_t projection_forest_forward_workspace(const ForestDims &d);
int projection_forest_forward(const ForestDims &d, bool fern, long long K_in, const float *x, const float *lin, double eps,
                              const float *thr, const int64_t *ord, const float *w, float *out, float *z, float *mean,
                              float *rstd, float *var, void *records, void *ws, size_t ws_bytes, hipStream_t stream);
size_t projection_forest_backward_workspace(const ForestDims &d, long long K_in);
int projection_forest_backward(const ForestDims &d, bool fern, long long K_in, const float *x, const float *lin,
                               const float *zhat, const float *mean, const float *rstd, const float *w, const float *gout,
                               const void *records, float *dthr, float *dw, float *dlin, void *ws, size_t ws_bytes,
                               hipStream_t stream);
// Host-side view of the matrix-product kernel's workgroup -> result-tile map for tiles_i x tiles_j tiles: writes the
// tile of every launch slot (-1, -1 for a slot without a tile) and returns the number of slots.
int gemm_tile_map(int tiles_i, int tiles_j, int *tile_i, int *tile_j);
int ordinal_range(const int64_t *ord, int64_t n, int64_t *minmax, hipStream_t stream);

// Lets `kernel` use all of a workgroup's LDS as dynamic shared memory. The runtime call behind it is made once per
// kernel and device, not per launch: later launches -- also those recorded into a HIP graph -- make no attribute
// calls at all.
hipError_t grant_lds(const void *kernel);

// Fills `bytes` bytes with zero through a kernel (safe to record into a HIP graph, unlike a memset node).
int zero_fill(void *p, size_t bytes, hipStream_t stream);

}  // namespace ht
