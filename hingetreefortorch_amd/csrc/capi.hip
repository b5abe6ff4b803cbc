// extern "C" surface of libhingetree_hip.so (declared in include/hingetree_hip.h) and the host-only pieces.
#include <cmath>
#include <cstring>
#include <limits>
#include <mutex>
#include <set>
#include <utility>

#include "common.hpp"

// Workspace of ht_forest_forward_static (the forward pass for callers that cannot allocate): one array per GPU, part
// of the library's code object, held by every GPU the library runs on until the process ends. In host code the array's
// name is only a handle for hipGetSymbolAddress; the device address that call yields (one per device) is what the
// kernels and the packing pre-passes receive.
static __device__ __align__(256) unsigned char scratch[HT_STATIC_SCRATCH_BYTES];

namespace ht {

static thread_local std::string g_last_error;

void set_error(const std::string &msg) { g_last_error = msg; }
int fail(int code, const std::string &msg) {
  g_last_error = msg;
  return code;
}

// Shape rules and messages of hingetree.cpp:66-94 that can be decided from sizes alone.
int make_dims(const ht_forest_shape *s, ForestDims *d) {
  if (!s) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null shape.");
  if (s->dtype != HT_F32 && s->dtype != HT_F64)
    return fail(HT_ERR_INVALID_ARGUMENT,
                "Error: Unsupported data type. Only torch.float32 and torch.float64 are supported.");
  if (s->kind != HT_TREE && s->kind != HT_FERN) return fail(HT_ERR_INVALID_ARGUMENT, "Error: unknown tree kind.");
  if (s->depth < 1 || s->depth > 31)  // 32-bit leaf keys, HingeTreeCommon.h:51,138; a depth-0 walk reads no vertex
    return fail(HT_ERR_RUNTIME,
                "Error: The tree depth exceeds compile-time constraints or the number of thresholds is incorrect for "
                "the tree depth (tree depth = " + std::to_string((long long)s->depth) + ").");
  if (s->B < 0 || s->F < 0 || s->K < 0 || s->T < 0 || s->M < 0)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: negative tensor size.");
  const long long V = s->kind == HT_FERN ? s->depth : ((1LL << s->depth) - 1), L = 1LL << s->depth;
  const long long lim = 0x7fffffffLL;
  if (s->F > lim || s->K > lim || s->T > lim || s->M > lim || V > lim || L > lim || L * s->M > lim)
    return fail(HT_ERR_RUNTIME, "Error: a tensor dimension exceeds the 32-bit limits of this build.");
  if (s->depth > 0 && V == 0) return fail(HT_ERR_RUNTIME, "Error: inconsistent tree shape.");
  d->S = s->B * s->K;
  d->FK = s->F * s->K;
  d->F = int(s->F);
  d->K = int(s->K);
  d->T = int(s->T);
  d->depth = int(s->depth);
  d->V = int(V);
  d->L = int(L);
  d->M = int(s->M);
  return HT_OK;
}

int make_image_store(const ht_tile_shape *g, const ForestDims &d, long long B, ImageStore *img, bool *clear) {
  if (!g) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null shape.");
  if (g->nd != 2 && g->nd != 3)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: Only 2D and 3D window sizes are supported.");
  const int shift = 3 - g->nd;  // a 2-d geometry is a 3-d one with a leading dimension of extent 1
  for (int dd = 0; dd < 3; ++dd) {
    img->tiles[dd] = img->win[dd] = img->size[dd] = 1;
    img->pad[dd] = 0;
  }
  long long positions = 1, outputs = 1, plane = 1;
  *clear = false;
  for (int dd = 0; dd < g->nd; ++dd) {
    if (g->size[dd] < 1 || g->tiles[dd] < 1 || g->window[dd] < 1 || g->padding[dd] < 0 || g->size[dd] > 0x3fffffff ||
        g->tiles[dd] > 0x3fffffff || g->window[dd] > 0x3fffffff || g->padding[dd] > 0x3fffffff)
      return fail(HT_ERR_INVALID_ARGUMENT, "Error: invalid tile geometry.");
    img->size[dd + shift] = int(g->size[dd]);
    img->tiles[dd + shift] = int(g->tiles[dd]);
    img->win[dd + shift] = int(g->window[dd]);
    img->pad[dd + shift] = int(g->padding[dd]);
    positions *= g->tiles[dd];
    outputs *= g->window[dd];
    plane *= g->size[dd];
    if (g->size[dd] > g->tiles[dd] * g->window[dd] - g->padding[dd]) *clear = true;  // positions behind the last tile
  }
  if (positions != d.K || outputs != d.M || g->planes != B * d.T)
    return fail(HT_ERR_INVALID_ARGUMENT,
                "Error: the tile geometry does not match the forest (tiles = inner data positions, window = outputs "
                "per leaf, planes = samples x trees).");
  if (plane > (1ll << 40)) return fail(HT_ERR_RUNTIME, "Error: image too large for this build.");
  // the in-kernel divisions are exact for dividend x divisor < 2^32
  for (int dd = 1; dd < 3; ++dd)
    if ((long long)d.K * img->tiles[dd] >= (1ll << 32) || (long long)d.M * img->win[dd] >= (1ll << 32))
      return fail(HT_ERR_RUNTIME, "Error: tile geometry too large for the image store of this build.");
  for (int dd = 0; dd < 3; ++dd) {
    img->by_tiles[dd] = FastDiv(img->tiles[dd]);
    img->by_win[dd] = FastDiv(img->win[dd]);
  }
  img->plane = plane;
  img->nd = g->nd;
  return HT_OK;
}

// ---- threshold consistency (host memory) -----------------------------------------------------------------------
// A vertex that re-tests a feature already tested by an ancestor must keep its threshold on the side of the ancestor's
// threshold that its path came from (HingeTreeCommon.h:211-287).
template <typename Real>
static bool tree_consistent(const Real *thr, const int64_t *ord, int64_t V) {
  for (int64_t i = V - 1; i > 0; --i) {
    int64_t child = i;
    while (child > 0) {
      const int64_t up = (child - 1) >> 1;
      if (ord[up] == ord[i]) {
        const bool from_right = (child & 1) == 0;  // right children have even heap indices
        if (from_right ? thr[i] < thr[up] : thr[i] > thr[up]) return false;
      }
      child = up;
    }
  }
  return true;
}

template <typename Real>
static bool tree_repair(Real *thr, const int64_t *ord, int64_t V) {
  bool changed = false;
  const Real inf = std::numeric_limits<Real>::infinity();
  for (int64_t i = 1; i < V; ++i) {
    Real lower = -inf, upper = inf;
    int64_t child = i;
    while (child > 0) {
      const int64_t up = (child - 1) >> 1;
      if (ord[up] == ord[i]) {
        if ((child & 1) == 0)
          lower = std::max(lower, thr[up]);
        else
          upper = std::min(upper, thr[up]);
      }
      child = up;
    }
    if (thr[i] < lower || thr[i] > upper) {
      if (!std::isfinite(lower))
        thr[i] = upper - Real(1);
      else if (!std::isfinite(upper))
        thr[i] = lower + Real(1);
      else
        thr[i] = Real(0.5) * (lower + upper);
      changed = true;
    }
  }
  return changed;
}

// ---- the static workspace's device address, per device -------------------------------------------------------------
constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void *g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (looked up once per device, with that device current).
static int static_scratch(void **ptr) {
  int dev = -1;
  HT_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(HT_ERR_RUNTIME, "Error: device index beyond the static workspace table.");
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    HT_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(HT_ERR_HIP, "hipGetSymbolAddress returned a null address for the static workspace.");
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return HT_OK;
}

// ---- dynamic LDS limit of a kernel, granted once per kernel and device -------------------------------------------
hipError_t grant_lds(const void *kernel) {
  static std::mutex mutex;
  static std::set<std::pair<int, const void *>> granted;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  std::lock_guard<std::mutex> lock(mutex);
  const std::pair<int, const void *> key(dev, kernel);
  if (granted.count(key)) return hipSuccess;
  hipFuncAttributes attr;
  if ((e = hipFuncGetAttributes(&attr, kernel)) != hipSuccess) return e;
  const int room = kLdsBytes - int(attr.sharedSizeBytes);  // what the kernel's static arrays leave
  if ((e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, room)) != hipSuccess) return e;
  granted.insert(key);
  return hipSuccess;
}

}  // namespace ht

using namespace ht;

extern "C" {

const char *ht_last_error(void) { return g_last_error.c_str(); }
int ht_abi_version(void) { return HT_ABI_VERSION; }

int ht_check_device(int32_t device) {
  hipDeviceProp_t prop;
  HT_HIP_CHECK(hipGetDeviceProperties(&prop, device));
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(HT_ERR_RUNTIME, std::string("Error: this library holds kernels for gfx950 (MI355X) only; device ") +
                                    std::to_string(device) + " is " + prop.gcnArchName + ".");
  return HT_OK;
}

int ht_ordinal_range(const int64_t *ord, int64_t n, int64_t *minmax, void *stream) {
  if (!minmax || (n > 0 && !ord)) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  return ordinal_range(ord, n, minmax, static_cast<hipStream_t>(stream));
}

size_t ht_forest_forward_workspace(const ht_forest_shape *s) {
  ForestDims d;
  if (make_dims(s, &d) != HT_OK) return 0;
  return s->dtype == HT_F32 ? forest_forward_workspace<float>(d) : forest_forward_workspace<double>(d);
}

int ht_forest_forward(const ht_forest_shape *s, const void *x, const void *thr, const int64_t *ord, const void *w,
                      void *out, void *workspace, size_t workspace_bytes, void *stream) {
  ForestDims d;
  int rc = make_dims(s, &d);
  if (rc != HT_OK) return rc;
  if (!is_empty(d) && (!x || !thr || !ord || !w || !out))
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool fern = s->kind == HT_FERN;
  if (s->dtype == HT_F32)
    return forest_forward<float>(d, fern, (const float *)x, (const float *)thr, ord, (const float *)w, (float *)out,
                                 nullptr, workspace, workspace_bytes, st);
  return forest_forward<double>(d, fern, (const double *)x, (const double *)thr, ord, (const double *)w, (double *)out,
                                nullptr, workspace, workspace_bytes, st);
}

int ht_forest_forward_static(const ht_forest_shape *s, const void *x, const void *thr, const int64_t *ord,
                             const void *w, void *out, void *stream) {
  ForestDims d;
  int rc = make_dims(s, &d);
  if (rc != HT_OK) return rc;
  const size_t need = ht_forest_forward_workspace(s);
  if (need > size_t(HT_STATIC_SCRATCH_BYTES))
    return fail(HT_ERR_INVALID_ARGUMENT,
                "Error: this forest needs " + std::to_string(need) + " bytes of workspace, more than the " +
                    std::to_string(size_t(HT_STATIC_SCRATCH_BYTES)) +
                    " bytes ht_forest_forward_static holds; call ht_forest_forward with a workspace of your own.");
  void *ws = nullptr;
  if ((rc = static_scratch(&ws)) != HT_OK) return rc;  // also for an empty shape: a caller's set-up call
  if (is_empty(d)) return HT_OK;
  if (!x || !thr || !ord || !w || !out) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool fern = s->kind == HT_FERN;
  if (s->dtype == HT_F32)
    return forest_forward<float>(d, fern, (const float *)x, (const float *)thr, ord, (const float *)w, (float *)out,
                                 nullptr, ws, size_t(HT_STATIC_SCRATCH_BYTES), st);
  return forest_forward<double>(d, fern, (const double *)x, (const double *)thr, ord, (const double *)w, (double *)out,
                                nullptr, ws, size_t(HT_STATIC_SCRATCH_BYTES), st);
}

int ht_forest_forward_image(const ht_forest_shape *s, const ht_tile_shape *g, const void *x, const void *thr,
                            const int64_t *ord, const void *w, void *image, void *workspace, size_t workspace_bytes,
                            void *stream) {
  ForestDims d;
  int rc = make_dims(s, &d);
  if (rc != HT_OK) return rc;
  ImageStore img{};
  bool clear = false;
  if ((rc = make_image_store(g, d, s->B, &img, &clear)) != HT_OK) return rc;
  if (g->elem_size != (s->dtype == HT_F32 ? 4 : 8))
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: the element size of the tile geometry must be that of the forest's data type.");
  if (d.K == 1)
    return fail(HT_ERR_INVALID_ARGUMENT,
                "Error: an image result needs inner data positions (inData of 3 or more dimensions).");
  if (is_empty(d)) return HT_OK;
  if (!x || !thr || !ord || !w || !image) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (clear && (rc = zero_fill(image, size_t(g->planes) * size_t(img.plane) * size_t(g->elem_size), st)) != HT_OK)
    return rc;
  const bool fern = s->kind == HT_FERN;
  if (s->dtype == HT_F32)
    return forest_forward<float>(d, fern, (const float *)x, (const float *)thr, ord, (const float *)w, (float *)image,
                                 nullptr, workspace, workspace_bytes, st, &img);
  return forest_forward<double>(d, fern, (const double *)x, (const double *)thr, ord, (const double *)w,
                                (double *)image, nullptr, workspace, workspace_bytes, st, &img);
}

size_t ht_forest_records_bytes(const ht_forest_shape *s) {
  ForestDims d;
  if (make_dims(s, &d) != HT_OK) return 0;
  return s->dtype == HT_F32 ? forest_records_bytes<float>(d) : forest_records_bytes<double>(d);
}

int ht_forest_forward_records(const ht_forest_shape *s, const void *x, const void *thr, const int64_t *ord,
                              const void *w, void *out, void *records, size_t records_bytes, void *workspace,
                              size_t workspace_bytes, void *stream) {
  ForestDims d;
  int rc = make_dims(s, &d);
  if (rc != HT_OK) return rc;
  const size_t need = ht_forest_records_bytes(s);
  if (need == 0 && !is_empty(d))
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: walk records are not offered for this shape.");
  if (!is_empty(d) && (!x || !thr || !ord || !w || !out || !records))
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  if (records_bytes < need) return fail(HT_ERR_INVALID_ARGUMENT, "Error: records buffer too small.");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool fern = s->kind == HT_FERN;
  if (s->dtype == HT_F32)
    return forest_forward<float>(d, fern, (const float *)x, (const float *)thr, ord, (const float *)w, (float *)out,
                                 records, workspace, workspace_bytes, st);
  return forest_forward<double>(d, fern, (const double *)x, (const double *)thr, ord, (const double *)w, (double *)out,
                                records, workspace, workspace_bytes, st);
}

size_t ht_forest_backward_records_workspace(const ht_forest_shape *s, int mode, int need_dx, int need_dthr,
                                            int need_dw) {
  ForestDims d;
  if (make_dims(s, &d) != HT_OK) return 0;
  return s->dtype == HT_F32
             ? forest_backward_records_workspace<float>(d, mode, need_dx != 0, need_dthr != 0, need_dw != 0)
             : forest_backward_records_workspace<double>(d, mode, need_dx != 0, need_dthr != 0, need_dw != 0);
}

int ht_forest_backward_records(const ht_forest_shape *s, const void *w, const void *gout, const void *records,
                               size_t records_bytes, void *dx, void *dthr, void *dw, int mode, void *workspace,
                               size_t workspace_bytes, void *stream) {
  ForestDims d;
  int rc = make_dims(s, &d);
  if (rc != HT_OK) return rc;
  if (mode != HT_BACKWARD_ATOMIC && mode != HT_BACKWARD_DETERMINISTIC)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: unknown backward mode.");
  const size_t need = ht_forest_records_bytes(s);
  if (need == 0 && !is_empty(d))
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: walk records are not offered for this shape.");
  if (!is_empty(d) && (!w || !gout || !records)) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  if (records_bytes < need) return fail(HT_ERR_INVALID_ARGUMENT, "Error: records buffer too small.");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool fern = s->kind == HT_FERN;
  if (s->dtype == HT_F32)
    return forest_backward_records<float>(d, fern, (const float *)w, (const float *)gout, records, (float *)dx,
                                          (float *)dthr, (float *)dw, mode, workspace, workspace_bytes, st);
  return forest_backward_records<double>(d, fern, (const double *)w, (const double *)gout, records, (double *)dx,
                                         (double *)dthr, (double *)dw, mode, workspace, workspace_bytes, st);
}

size_t ht_forest_backward_workspace(const ht_forest_shape *s, int mode, int need_dx, int need_dthr, int need_dw) {
  ForestDims d;
  if (make_dims(s, &d) != HT_OK) return 0;
  return s->dtype == HT_F32 ? forest_backward_workspace<float>(d, mode, need_dx != 0, need_dthr != 0, need_dw != 0)
                            : forest_backward_workspace<double>(d, mode, need_dx != 0, need_dthr != 0, need_dw != 0);
}

int ht_forest_backward(const ht_forest_shape *s, const void *x, const void *thr, const int64_t *ord, const void *w,
                       const void *gout, void *dx, void *dthr, void *dw, int mode, void *workspace,
                       size_t workspace_bytes, void *stream) {
  ForestDims d;
  int rc = make_dims(s, &d);
  if (rc != HT_OK) return rc;
  if (mode != HT_BACKWARD_ATOMIC && mode != HT_BACKWARD_DETERMINISTIC)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: unknown backward mode.");
  if (!is_empty(d) && (!x || !thr || !ord || !w || !gout))
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool fern = s->kind == HT_FERN;
  if (s->dtype == HT_F32)
    return forest_backward<float>(d, fern, (const float *)x, (const float *)thr, ord, (const float *)w,
                                  (const float *)gout, (float *)dx, (float *)dthr, (float *)dw, mode, workspace,
                                  workspace_bytes, st);
  return forest_backward<double>(d, fern, (const double *)x, (const double *)thr, ord, (const double *)w,
                                 (const double *)gout, (double *)dx, (double *)dthr, (double *)dw, mode, workspace,
                                 workspace_bytes, st);
}

static int image_backward_geometry(const ht_forest_shape *s, const ht_tile_shape *g, ForestDims *d, ImageStore *img) {
  int rc = make_dims(s, d);
  if (rc != HT_OK) return rc;
  bool clear = false;
  if ((rc = make_image_store(g, *d, s->B, img, &clear)) != HT_OK) return rc;
  if (g->elem_size != (s->dtype == HT_F32 ? 4 : 8))
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: the element size of the tile geometry must be that of the forest's data type.");
  return HT_OK;
}

int ht_forest_backward_image_supported(const ht_forest_shape *s, const ht_tile_shape *g, int mode, int need_dx,
                                       int need_dthr, int need_dw) {
  (void)need_dthr;
  ForestDims d;
  ImageStore img{};
  if (image_backward_geometry(s, g, &d, &img) != HT_OK) return 0;
  if (s->dtype != HT_F32) return 0;
  return forest_backward_image_ok<float>(d, mode, need_dx != 0, need_dw != 0, img) ? 1 : 0;
}

int ht_forest_backward_image(const ht_forest_shape *s, const ht_tile_shape *g, const void *x, const void *thr,
                             const int64_t *ord, const void *w, const void *gout_image, void *dx, void *dthr, void *dw,
                             int mode, void *workspace, size_t workspace_bytes, void *stream) {
  ForestDims d;
  ImageStore img{};
  int rc = image_backward_geometry(s, g, &d, &img);
  if (rc != HT_OK) return rc;
  if (mode != HT_BACKWARD_ATOMIC && mode != HT_BACKWARD_DETERMINISTIC)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: unknown backward mode.");
  if (!is_empty(d) && (!x || !thr || !ord || !w || !gout_image))
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  if (!is_empty(d) && (s->dtype != HT_F32 || !forest_backward_image_ok<float>(d, mode, dx != nullptr, dw != nullptr, img)))
    return fail(HT_ERR_INVALID_ARGUMENT,
                "Error: this shape, data type or mode cannot read the upstream gradient as an image (ask "
                "ht_forest_backward_image_supported; contract the gradient and call ht_forest_backward instead).");
  return forest_backward<float>(d, s->kind == HT_FERN, (const float *)x, (const float *)thr, ord, (const float *)w,
                                (const float *)gout_image, (float *)dx, (float *)dthr, (float *)dw, mode, workspace,
                                workspace_bytes, static_cast<hipStream_t>(stream), &img);
}

size_t ht_forest_maps_workspace(const ht_forest_shape *s, int32_t want_reach) {
  ForestDims d;
  if (make_dims(s, &d) != HT_OK) return 0;
  return s->dtype == HT_F32 ? forest_maps_workspace<float>(d, want_reach != 0)
                            : forest_maps_workspace<double>(d, want_reach != 0);
}

int ht_forest_maps(const ht_forest_shape *s, const void *x, const void *thr, const int64_t *ord, int64_t *leafmap,
                   void *margins, int64_t *ordinals, int64_t *reach, void *workspace, size_t workspace_bytes,
                   void *stream) {
  ForestDims d;
  int rc = make_dims(s, &d);
  if (rc != HT_OK) return rc;
  if (d.S > 0 && d.T > 0 && (!x || !thr || !ord)) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool fern = s->kind == HT_FERN;
  if (s->dtype == HT_F32)
    return forest_maps<float>(d, fern, (const float *)x, (const float *)thr, ord, leafmap, (float *)margins, ordinals,
                              reach, workspace, workspace_bytes, st);
  return forest_maps<double>(d, fern, (const double *)x, (const double *)thr, ord, leafmap, (double *)margins, ordinals,
                             reach, workspace, workspace_bytes, st);
}

static int check_conv(const ht_conv_shape *s) {
  if (!s) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null shape.");
  if (s->dtype != HT_F32 && s->dtype != HT_F64)
    return fail(HT_ERR_INVALID_ARGUMENT,
                "Error: Unsupported data type. Only torch.float32 and torch.float64 are supported.");
  if (s->depth < 0 || s->depth > 31)
    return fail(HT_ERR_RUNTIME,
                "Error: The tree depth exceeds compile-time constraints or the number of thresholds is incorrect for "
                "the tree depth (tree depth = " + std::to_string((long long)s->depth) + ").");
  if (s->B < 0 || s->C < 0 || s->Cout < 0 || s->M < 0) return fail(HT_ERR_INVALID_ARGUMENT, "Error: negative tensor size.");
  if ((1LL << s->depth) * s->M > 0x7fffffffLL || s->C > 0x7fffffffLL)
    return fail(HT_ERR_RUNTIME, "Error: a tensor dimension exceeds the 32-bit limits of this build.");
  return HT_OK;
}

int ht_conv_output_size(const ht_conv_shape *s, int64_t *out_size) {
  int rc = check_conv(s);
  if (rc != HT_OK) return rc;
  return conv_output_size(*s, out_size);
}

int ht_conv_forward(const ht_conv_shape *s, const void *x, const void *thr, const int64_t *ord, const void *w, void *out,
                    void *stream) {
  int rc = check_conv(s);
  if (rc != HT_OK) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (s->dtype == HT_F32)
    return conv_forward<float>(*s, (const float *)x, (const float *)thr, ord, (const float *)w, (float *)out, st);
  return conv_forward<double>(*s, (const double *)x, (const double *)thr, ord, (const double *)w, (double *)out, st);
}

int ht_conv_backward(const ht_conv_shape *s, const void *x, const void *thr, const int64_t *ord, const void *w,
                     const void *gout, void *dx, void *dthr, void *dw, void *stream) {
  int rc = check_conv(s);
  if (rc != HT_OK) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (s->dtype == HT_F32)
    return conv_backward<float>(*s, (const float *)x, (const float *)thr, ord, (const float *)w, (const float *)gout,
                                (float *)dx, (float *)dthr, (float *)dw, st);
  return conv_backward<double>(*s, (const double *)x, (const double *)thr, ord, (const double *)w, (const double *)gout,
                               (double *)dx, (double *)dthr, (double *)dw, st);
}

static int thresholds_common(int64_t T, int64_t depth, int32_t dtype, int32_t kind, int64_t *V) {
  if (dtype != HT_F32 && dtype != HT_F64)
    return fail(HT_ERR_INVALID_ARGUMENT,
                "Error: Unsupported data type. Only torch.float32 and torch.float64 are supported.");
  if (T < 0 || depth < 0 || depth > 31) return fail(HT_ERR_RUNTIME, "Error: invalid tree shape.");
  *V = kind == HT_FERN ? depth : ((int64_t(1) << depth) - 1);
  return HT_OK;
}

int ht_tree_mix_forward(int64_t B, int64_t T, int64_t O, int64_t R, const float *f, const float *lin,
                        const float *bias, float *out, void *stream) {
  if (B < 0 || T < 0 || O < 0 || R < 0) return fail(HT_ERR_INVALID_ARGUMENT, "Error: negative tensor size.");
  if (B * O * R > 0 && (!out || (T > 0 && (!f || !lin)))) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  return mix_forward(B, T, O, R, f, lin, bias, out, static_cast<hipStream_t>(stream));
}

int ht_tree_mix_backward(int64_t B, int64_t T, int64_t O, int64_t R, const float *f, const float *lin, const float *g,
                         float *h, float *dlin, int deterministic, void *stream) {
  if (B < 0 || T < 0 || O < 0 || R < 0) return fail(HT_ERR_INVALID_ARGUMENT, "Error: negative tensor size.");
  if (B * O * R > 0 && (!g || (h && !lin) || (dlin && !f))) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  return mix_backward(B, T, O, R, f, lin, g, h, dlin, deterministic != 0, static_cast<hipStream_t>(stream));
}

size_t ht_tree_mix_backward_workspace(int64_t B, int64_t T, int64_t O, int64_t R) {
  return (B < 0 || T < 0 || O < 0 || R < 0) ? 0 : mix_backward_workspace(B, T, O, R);
}

int ht_tree_mix_backward_ws(int64_t B, int64_t T, int64_t O, int64_t R, const float *f, const float *lin, const float *g,
                            float *h, float *dlin, int deterministic, void *workspace, size_t workspace_bytes,
                            void *stream) {
  if (B < 0 || T < 0 || O < 0 || R < 0) return fail(HT_ERR_INVALID_ARGUMENT, "Error: negative tensor size.");
  if (B * O * R > 0 && (!g || (h && !lin) || (dlin && !f))) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  return mix_backward(B, T, O, R, f, lin, g, h, dlin, deterministic != 0, static_cast<hipStream_t>(stream), workspace,
                      workspace_bytes);
}

int ht_rows_to_planes(int64_t n, int64_t R, const float *rows, float *planes, void *stream) {
  if (n < 0 || R < 0) return fail(HT_ERR_INVALID_ARGUMENT, "Error: negative tensor size.");
  if (n > 0 && R > 0 && (!rows || !planes)) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  return rows_to_planes(n, R, rows, planes, false, static_cast<hipStream_t>(stream));
}

int ht_planes_to_rows(int64_t n, int64_t R, const float *planes, float *rows, void *stream) {
  if (n < 0 || R < 0) return fail(HT_ERR_INVALID_ARGUMENT, "Error: negative tensor size.");
  if (n > 0 && R > 0 && (!rows || !planes)) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  return rows_to_planes(n, R, planes, rows, true, static_cast<hipStream_t>(stream));
}

int ht_tree_mix_forward_f64(int64_t B, int64_t T, int64_t O, int64_t R, const double *f, const double *lin,
                            const double *bias, double *out, void *stream) {
  if (B < 0 || T < 0 || O < 0 || R < 0) return fail(HT_ERR_INVALID_ARGUMENT, "Error: negative tensor size.");
  if (B * O * R > 0 && (!out || (T > 0 && (!f || !lin)))) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  return mix_forward_f64(B, T, O, R, f, lin, bias, out, static_cast<hipStream_t>(stream));
}

int ht_tree_mix_backward_f64(int64_t B, int64_t T, int64_t O, int64_t R, const double *f, const double *lin,
                             const double *g, double *h, double *dlin, void *stream) {
  if (B < 0 || T < 0 || O < 0 || R < 0) return fail(HT_ERR_INVALID_ARGUMENT, "Error: negative tensor size.");
  if (B * O * R > 0 && (!g || (h && !lin) || (dlin && !f))) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  return mix_backward_f64(B, T, O, R, f, lin, g, h, dlin, static_cast<hipStream_t>(stream));
}

int ht_contract(const ht_tile_shape *s, const void *image, void *tiles, void *stream) {
  if (s && s->planes > 0 && (!image || !tiles)) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  return tile_contract(s, image, tiles, static_cast<hipStream_t>(stream));
}

int ht_expand(const ht_tile_shape *s, const void *tiles, void *image, void *stream) {
  if (s && s->planes > 0 && (!image || !tiles)) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  return tile_expand(s, tiles, image, static_cast<hipStream_t>(stream));
}

size_t ht_projection_workspace(int64_t N) { return N < 0 ? 0 : projection_workspace(N); }
size_t ht_projection_backward_workspace(int64_t B, int64_t K, int64_t N) {
  return (B < 0 || K < 0 || N < 0) ? 0 : projection_backward_workspace(B, K, N);
}

int ht_projection_forward(int64_t B, int64_t K, int64_t N, const float *x, const float *lin, double eps, float *zhat,
                          float *mean, float *rstd, float *var, void *workspace, size_t workspace_bytes, void *stream) {
  if (B < 0 || K < 0 || N < 0) return fail(HT_ERR_INVALID_ARGUMENT, "Error: negative tensor size.");
  if (N > 0 && (!mean || !rstd || !workspace)) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  if (B > 0 && N > 0 && (!zhat || (K > 0 && (!x || !lin)))) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  if (workspace_bytes < projection_workspace(N))
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: workspace too small for the projection.");
  return projection_forward(B, K, N, x, lin, eps, zhat, mean, rstd, var, workspace, static_cast<hipStream_t>(stream));
}

int ht_projection_backward(int64_t B, int64_t K, int64_t N, const float *x, const float *lin, const float *zhat,
                           const float *rstd, float *g, float *dlin, float *dx, void *workspace,
                           size_t workspace_bytes, void *stream) {
  if (B < 0 || K < 0 || N < 0) return fail(HT_ERR_INVALID_ARGUMENT, "Error: negative tensor size.");
  if (B > 0 && N > 0 && (!zhat || !rstd || !g || !workspace || (dlin && !x) || (dx && !lin)))
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  if (workspace_bytes < projection_backward_workspace(B, K, N))
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: workspace too small for the projection.");
  return projection_backward(B, K, N, x, lin, zhat, rstd, g, dlin, dx, workspace, static_cast<hipStream_t>(stream));
}

size_t ht_projection_forest_backward_workspace(const ht_forest_shape *forest, int64_t K_in) {
  ForestDims d;
  if (!forest || forest->dtype != HT_F32 || make_dims(forest, &d) != HT_OK) return 0;
  return projection_forest_backward_workspace(d, K_in);
}

size_t ht_projection_forest_forward_workspace(const ht_forest_shape *forest) {
  ForestDims d;
  if (!forest || forest->dtype != HT_F32 || forest->K != 1 || make_dims(forest, &d) != HT_OK) return 0;
  return projection_forest_forward_workspace(d);
}

int ht_projection_forest_forward(const ht_forest_shape *forest, int64_t K_in, const float *x, const float *lin, double eps,
                                 const float *thr, const int64_t *ord, const float *w, float *out, float *z, float *mean,
                                 float *rstd, float *var, void *records, size_t records_bytes, void *workspace,
                                 size_t workspace_bytes, void *stream) {
  ForestDims d;
  if (!forest) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  int rc = make_dims(forest, &d);
  if (rc != HT_OK) return rc;
  if (forest->dtype != HT_F32) return fail(HT_ERR_INVALID_ARGUMENT, "Error: the projection supports float32 only.");
  if (forest->K != 1 || K_in < 0)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: the projection's forest has no inner data dimensions.");
  if (d.F > 0 && (!mean || !rstd || !workspace)) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  if (d.S > 0 && d.F > 0 && (!z || (K_in > 0 && (!x || !lin)))) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  if (!is_empty(d) && (!thr || !ord || !w || !out)) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  if (records) {
    const size_t need = ht_forest_records_bytes(forest);
    if (need == 0 && !is_empty(d))
      return fail(HT_ERR_INVALID_ARGUMENT, "Error: walk records are not offered for this shape.");
    if (records_bytes < need) return fail(HT_ERR_INVALID_ARGUMENT, "Error: records buffer too small.");
  }
  return projection_forest_forward(d, forest->kind == HT_FERN, K_in, x, lin, eps, thr, ord, w, out, z, mean, rstd, var,
                                   records, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int ht_projection_forest_backward(const ht_forest_shape *forest, int64_t K_in, const float *x, const float *lin,
                                  const float *zhat, const float *mean, const float *rstd, const float *w, const float *gout,
                                  const void *records, size_t records_bytes, float *dthr, float *dw, float *dlin,
                                  void *workspace, size_t workspace_bytes, void *stream) {
  ForestDims d;
  if (!forest) return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  int rc = make_dims(forest, &d);
  if (rc != HT_OK) return rc;
  if (forest->dtype != HT_F32) return fail(HT_ERR_INVALID_ARGUMENT, "Error: the projection supports float32 only.");
  if (!projection_forest_backward_ok(d, K_in))
    return fail(HT_ERR_INVALID_ARGUMENT,
                "Error: this shape is not served by the records form of the projection backward "
                "(ht_projection_forest_backward_workspace returns 0 for it).");
  if (!x || !lin || !zhat || !rstd || !w || !gout || !records || !workspace)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: null pointer.");
  if (records_bytes < ht_forest_records_bytes(forest))
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: records buffer too small.");
  return projection_forest_backward(d, forest->kind == HT_FERN, K_in, x, lin, zhat, mean, rstd, w, gout, records, dthr, dw,
                                    dlin, workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int ht_gemm_tile_map(int32_t tiles_i, int32_t tiles_j, int32_t *tile_i, int32_t *tile_j, int64_t capacity) {
  if (tiles_i < 1 || tiles_j < 1) return fail(HT_ERR_INVALID_ARGUMENT, "Error: a tile grid needs at least one tile.");
  const long long slots = (long long)((tiles_i + kNumXCDs - 1) / kNumXCDs) * tiles_j * kNumXCDs;
  if (!tile_i || !tile_j || capacity < slots)
    return fail(HT_ERR_INVALID_ARGUMENT, "Error: the tile map needs room for " + std::to_string(slots) + " launch slots.");
  gemm_tile_map(tiles_i, tiles_j, tile_i, tile_j);
  return HT_OK;
}

int ht_check_thresholds(const void *thr, const int64_t *ord, int64_t T, int64_t depth, int32_t dtype, int32_t kind,
                        uint8_t *flags) {
  int64_t V;
  int rc = thresholds_common(T, depth, dtype, kind, &V);
  if (rc != HT_OK) return rc;
  for (int64_t t = 0; t < T; ++t) {
    if (kind == HT_FERN)
      flags[t] = 1;
    else if (dtype == HT_F32)
      flags[t] = tree_consistent<float>((const float *)thr + t * V, ord + t * V, V);
    else
      flags[t] = tree_consistent<double>((const double *)thr + t * V, ord + t * V, V);
  }
  return HT_OK;
}

int ht_fix_thresholds(void *thr, const int64_t *ord, int64_t T, int64_t depth, int32_t dtype, int32_t kind,
                      uint8_t *flags) {
  int64_t V;
  int rc = thresholds_common(T, depth, dtype, kind, &V);
  if (rc != HT_OK) return rc;
  for (int64_t t = 0; t < T; ++t) {
    if (kind == HT_FERN)
      flags[t] = 0;
    else if (dtype == HT_F32)
      flags[t] = tree_repair<float>((float *)thr + t * V, ord + t * V, V);
    else
      flags[t] = tree_repair<double>((double *)thr + t * V, ord + t * V, V);
  }
  return HT_OK;
}

}  // extern "C"
