// Native host of the operator module: a pybind11 / ATen extension that sits where the reference's own
// PYBIND11_MODULE does (hingetree.cpp:1962-2031) and drives libhingetree_hip.so through its C ABI
// (include/hingetree_hip.h). It exports the reference's operator names for the forest / fern / convolution path with
// the reference's positional signatures, validation order, exception types and messages (hingetree.cpp:66-94,
// 159-222, 648-1358; hingetree_conv.cpp:58-122,235-332), allocates outputs and scratch from torch's caching allocator
// on the inputs' device, launches on torch's current stream of that device under a device guard, and holds no state
// besides the remembered ordinal range checks.
//
// This file contains no kernels and nothing of the reference's sources; it is compiled with the host compiler against
// the installed torch headers and linked to libhingetree_hip.so.
#include <ATen/hip/HIPContext.h>
#include <c10/core/DeviceGuard.h>
#include <torch/extension.h>

#include <atomic>
#include <mutex>
#include <sstream>
#include <stdexcept>
#include <unordered_map>
#include <vector>

#include "../../include/hingetree_hip.h"

namespace {

[[noreturn]] void invalid(const std::string &msg) { throw std::invalid_argument(msg); }  // -> Python ValueError
[[noreturn]] void runtime(const std::string &msg) { throw std::runtime_error(msg); }     // -> Python RuntimeError

void check(int rc) {
  if (rc == HT_OK) return;
  const std::string msg = ht_last_error();
  if (rc == HT_ERR_INVALID_ARGUMENT) invalid(msg);
  runtime(msg);
}

int64_t prod(c10::IntArrayRef v, size_t from) {
  int64_t r = 1;
  for (size_t i = from; i < v.size(); ++i) r *= v[i];
  return r;
}

// HingeTreeCommon.h:55-65,141-151: -1 unless the leaf count is a positive power of two
int64_t compute_depth(int64_t leaves) {
  if (leaves <= 0 || (leaves & (leaves - 1)) != 0) return -1;
  int64_t d = 0;
  while ((int64_t(1) << d) < leaves) ++d;
  return d;
}

[[noreturn]] void depth_error(int64_t depth) {
  std::ostringstream s;
  s << "Error: The tree depth exceeds compile-time constraints or the number of thresholds is incorrect for the tree "
       "depth (tree depth = "
    << depth << ").";
  runtime(s.str());
}

int dtype_code(const torch::Tensor &t) { return t.scalar_type() == torch::kFloat32 ? HT_F32 : HT_F64; }

void *ptr(const torch::Tensor &t) { return t.defined() ? t.data_ptr() : nullptr; }

// The stream torch is using on the tensor's device; the first use of a device also asks the library whether it can run
// there.
void *current_stream(const torch::Tensor &t) {
  static std::atomic<bool> checked[64];
  const int index = t.device().index();
  if (index >= 0 && index < 64 && !checked[index].load(std::memory_order_acquire)) {
    check(ht_check_device(index));
    checked[index].store(true, std::memory_order_release);
  }
  return static_cast<void *>(at::hip::getCurrentHIPStream(t.device().index()).stream());
}

torch::Tensor workspace(size_t bytes, const torch::Tensor &like) {
  if (bytes == 0) return torch::Tensor();
  return torch::empty({int64_t(bytes)}, like.options().dtype(torch::kUInt8));
}

std::string sizes_text(c10::IntArrayRef v) {
  std::ostringstream s;
  s << "[";
  for (size_t i = 0; i < v.size(); ++i) s << (i ? ", " : "") << v[i];
  s << "]";
  return s.str();
}

// hingetree.cpp:649-663: data types, devices, contiguity -- in that order
void common_checks(const std::vector<const torch::Tensor *> &reals, const torch::Tensor &ordinals, bool with_grad) {
  const torch::Tensor &data = *reals[0];
  bool same = ordinals.scalar_type() == torch::kInt64;
  for (const torch::Tensor *t : reals) same = same && t->scalar_type() == data.scalar_type();
  if (!same) {
    if (with_grad)
      invalid("Error: inData, inThresholds, inWeights, outDataGrad are expected to share the same torch real number "
              "data type. inOrdinals is expected to be type torch.int64.");
    invalid("Error: inData, inThresholds, inWeights are expected to share the same torch real number data type. "
            "inOrdinals is expected to be type torch.int64.");
  }
  bool one_device = ordinals.device() == data.device();
  for (const torch::Tensor *t : reals) one_device = one_device && t->device() == data.device();
  if (!one_device) invalid("Error: All tensors are expected to be on the same device.");
  bool contiguous = ordinals.is_contiguous();
  for (const torch::Tensor *t : reals) contiguous = contiguous && t->is_contiguous();
  if (!contiguous) invalid("Error: All tensors are expected to be contiguous.");
  if (data.scalar_type() != torch::kFloat32 && data.scalar_type() != torch::kFloat64)
    invalid("Error: Unsupported data type. Only torch.float32 and torch.float64 are supported.");
}

void require_gpu(const torch::Tensor &t) {
  if (!t.is_cuda())
    runtime("Error: this build of hingetree_cpp has no CPU back-end (its only back-end is the HIP library for "
            "MI355X); move the tensors to a ROCm device.");
}

// ---- ordinal range check --------------------------------------------------------------------------------------
// The reference reduces inOrdinals to its min and max and reads them back on every call (hingetree.cpp:91,
// hingetree_gpu.cu:445). The same check runs here, but its verdict is remembered per tensor object, version counter,
// storage address and size, so a module's fixed `ordinals` parameter costs one device -> host read in its lifetime.
// The weak reference keeps a dead tensor's address from being mistaken for a new tensor. Writes through `.data`
// advance no counter: forget_ordinal_checks() drops every verdict; the kernels clamp ordinals in any case.
struct RangeVerdict {
  c10::weak_intrusive_ptr<c10::TensorImpl> who;
  uint32_t version;
  const void *data;
  int64_t numel;
  int64_t bound;  // proven: 0 <= ordinals < bound
};
std::mutex g_range_mutex;
std::unordered_map<const c10::TensorImpl *, RangeVerdict> g_range_ok;

void forget_ordinal_checks() {
  std::lock_guard<std::mutex> lock(g_range_mutex);
  g_range_ok.clear();
}

void validate_ordinals(const torch::Tensor &ordinals, int64_t limit) {
  const c10::TensorImpl *impl = ordinals.unsafeGetTensorImpl();
  const uint32_t version = ordinals.is_inference() ? 0u : ordinals._version();
  {
    std::lock_guard<std::mutex> lock(g_range_mutex);
    auto it = g_range_ok.find(impl);
    if (it != g_range_ok.end()) {
      const RangeVerdict &v = it->second;
      if (!v.who.expired() && v.version == version && v.data == ordinals.data_ptr() && v.numel == ordinals.numel() &&
          v.bound <= limit)
        return;
      g_range_ok.erase(it);
    }
  }
  int64_t bound = 0;
  if (ordinals.numel() > 0) {
    const c10::DeviceGuard guard(ordinals.device());
    torch::Tensor mm = torch::empty({2}, ordinals.options());
    check(ht_ordinal_range(static_cast<const int64_t *>(ordinals.data_ptr()), ordinals.numel(),
                           static_cast<int64_t *>(mm.data_ptr()), current_stream(ordinals)));
    torch::Tensor host = mm.cpu();
    const int64_t lo = host.data_ptr<int64_t>()[0], hi = host.data_ptr<int64_t>()[1];
    if (lo < 0 || hi >= limit)
      runtime("Error: An ordinal value is either negative or larger than or equal to the number of channels.");
    bound = hi + 1;
  }
  std::lock_guard<std::mutex> lock(g_range_mutex);
  if (g_range_ok.size() > 4096) {  // drop the verdicts of tensors that no longer exist
    for (auto it = g_range_ok.begin(); it != g_range_ok.end();) it = it->second.who.expired() ? g_range_ok.erase(it) : ++it;
  }
  g_range_ok.erase(impl);
  g_range_ok.emplace(impl, RangeVerdict{c10::weak_intrusive_ptr<c10::TensorImpl>(ordinals.getIntrusivePtr()), version,
                                        ordinals.data_ptr(), ordinals.numel(), bound});
}

// ---- forest / fern --------------------------------------------------------------------------------------------
// Shape rules of hingetree_cpu_forward / _backward (hingetree.cpp:66-94,164-222).
ht_forest_shape forest_shape(int kind, const torch::Tensor &inData, const torch::Tensor &inThresholds,
                             const torch::Tensor &inOrdinals, const torch::Tensor &inWeights,
                             const torch::Tensor *outDataGrad, std::vector<int64_t> *out_sizes) {
  if (inData.dim() < 2 || inThresholds.dim() != 2 || inOrdinals.dim() != 2 || inWeights.dim() < 2 ||
      (outDataGrad && outDataGrad->dim() < 2))
    invalid("Error: inData, inWeights must have at least 2 dimensions. inThresholds and inOrdinals must have 2 "
            "dimensions.");
  if (inThresholds.sizes() != inOrdinals.sizes() || inWeights.size(0) != inThresholds.size(0))
    invalid("Error: inThresholds and inOrdinals must be the same shape. inWeights.shape[0] must be the same as "
            "inThresholds.shape[0].");
  const int64_t depth = compute_depth(inWeights.size(1));
  const int64_t want = depth < 0 ? -1 : (kind == HT_FERN ? depth : (int64_t(1) << depth) - 1);
  if (depth > 31 || depth < 0 || inThresholds.size(1) != want) depth_error(depth);
  require_gpu(inData);
  validate_ordinals(inOrdinals, inData.size(1));
  ht_forest_shape s;
  s.B = inData.size(0);
  s.F = inData.size(1);
  s.K = prod(inData.sizes(), 2);
  s.T = inWeights.size(0);
  s.depth = depth;
  s.M = prod(inWeights.sizes(), 2);
  s.dtype = dtype_code(inData);
  s.kind = kind;
  out_sizes->assign({inData.size(0), inWeights.size(0)});
  out_sizes->insert(out_sizes->end(), inData.sizes().begin() + 2, inData.sizes().end());
  out_sizes->insert(out_sizes->end(), inWeights.sizes().begin() + 2, inWeights.sizes().end());
  if (outDataGrad && outDataGrad->sizes() != c10::IntArrayRef(*out_sizes))
    invalid("Error: outDataGrad.shape does not match the expected shape (" + sizes_text(outDataGrad->sizes()) +
            " != " + sizes_text(*out_sizes) + ").");
  return s;
}

torch::Tensor forest_forward(int kind, const torch::Tensor &inData, const torch::Tensor &inThresholds,
                             const torch::Tensor &inOrdinals, const torch::Tensor &inWeights) {
  common_checks({&inData, &inThresholds, &inWeights}, inOrdinals, false);
  std::vector<int64_t> out_sizes;
  const ht_forest_shape s = forest_shape(kind, inData, inThresholds, inOrdinals, inWeights, nullptr, &out_sizes);
  const c10::DeviceGuard guard(inData.device());
  torch::Tensor out = torch::empty(out_sizes, inData.options());
  const size_t bytes = ht_forest_forward_workspace(&s);
  torch::Tensor ws = workspace(bytes, inData);
  check(ht_forest_forward(&s, ptr(inData), ptr(inThresholds), static_cast<const int64_t *>(ptr(inOrdinals)),
                          ptr(inWeights), ptr(out), ptr(ws), bytes, current_stream(inData)));
  return out;
}

py::object optional(const torch::Tensor &t) { return t.defined() ? py::cast(t) : py::none(); }

py::list gradient_list(const torch::Tensor &dx, const torch::Tensor &dthr, const torch::Tensor &dw) {
  py::list r;
  r.append(optional(dx));
  r.append(optional(dthr));
  r.append(py::none());
  r.append(optional(dw));
  return r;
}

py::list forest_backward(int kind, int mode, const torch::Tensor &inData, bool bInDataGrad,
                         const torch::Tensor &inThresholds, bool bInThresholdsGrad, const torch::Tensor &inOrdinals,
                         bool bInOrdinalsGrad, const torch::Tensor &inWeights, bool bInWeightsGrad,
                         const torch::Tensor &outDataGrad) {
  common_checks({&inData, &inThresholds, &inWeights, &outDataGrad}, inOrdinals, true);
  if (bInOrdinalsGrad)  // hingetree.cpp:159-162
    runtime("Error: Gradient on inOrdinals is requested, but inOrdinals never has a gradient.");
  std::vector<int64_t> out_sizes;
  const ht_forest_shape s = forest_shape(kind, inData, inThresholds, inOrdinals, inWeights, &outDataGrad, &out_sizes);
  const c10::DeviceGuard guard(inData.device());
  torch::Tensor dx = bInDataGrad ? torch::empty_like(inData) : torch::Tensor();
  torch::Tensor dthr = bInThresholdsGrad ? torch::empty_like(inThresholds) : torch::Tensor();
  torch::Tensor dw = bInWeightsGrad ? torch::empty_like(inWeights) : torch::Tensor();
  const size_t bytes = ht_forest_backward_workspace(&s, mode, bInDataGrad, bInThresholdsGrad, bInWeightsGrad);
  torch::Tensor ws = workspace(bytes, inData);
  check(ht_forest_backward(&s, ptr(inData), ptr(inThresholds), static_cast<const int64_t *>(ptr(inOrdinals)),
                           ptr(inWeights), ptr(outDataGrad), ptr(dx), ptr(dthr), ptr(dw), mode, ptr(ws), bytes,
                           current_stream(inData)));
  return gradient_list(dx, dthr, dw);
}

// Forward that also returns the walk records for forest_backward_records (None where the library offers none). Not
// part of the reference's module: its backward walks the trees again (hingetree_gpu.cu:619-730).
py::tuple forest_forward_records(int kind, const torch::Tensor &inData, const torch::Tensor &inThresholds,
                                 const torch::Tensor &inOrdinals, const torch::Tensor &inWeights) {
  common_checks({&inData, &inThresholds, &inWeights}, inOrdinals, false);
  std::vector<int64_t> out_sizes;
  const ht_forest_shape s = forest_shape(kind, inData, inThresholds, inOrdinals, inWeights, nullptr, &out_sizes);
  const size_t rec_bytes = ht_forest_records_bytes(&s);
  if (rec_bytes == 0 || inData.numel() == 0 || inWeights.numel() == 0)
    return py::make_tuple(forest_forward(kind, inData, inThresholds, inOrdinals, inWeights), py::none());
  const c10::DeviceGuard guard(inData.device());
  torch::Tensor out = torch::empty(out_sizes, inData.options());
  torch::Tensor records = torch::empty({int64_t(rec_bytes)}, inData.options().dtype(torch::kUInt8));
  const size_t bytes = ht_forest_forward_workspace(&s);
  torch::Tensor ws = workspace(bytes, inData);
  check(ht_forest_forward_records(&s, ptr(inData), ptr(inThresholds), static_cast<const int64_t *>(ptr(inOrdinals)),
                                  ptr(inWeights), ptr(out), ptr(records), rec_bytes, ptr(ws), bytes,
                                  current_stream(inData)));
  return py::make_tuple(out, records);
}

py::list forest_backward_records(int kind, int mode, const torch::Tensor &records, const torch::Tensor &inData,
                                 bool bInDataGrad, const torch::Tensor &inThresholds, bool bInThresholdsGrad,
                                 const torch::Tensor &inOrdinals, bool bInOrdinalsGrad, const torch::Tensor &inWeights,
                                 bool bInWeightsGrad, const torch::Tensor &outDataGrad) {
  // the library reads `records` as raw bytes through a device pointer: anything but the byte buffer a forward pass
  // filled, on the data's device, is refused here instead of reaching a kernel
  if (!records.defined() || records.scalar_type() != torch::kUInt8 || !records.is_contiguous())
    invalid("Error: records must be the contiguous uint8 tensor a *_forward_records call returned.");
  if (records.device() != inData.device()) invalid("Error: records and inData are on different devices.");
  common_checks({&inData, &inThresholds, &inWeights, &outDataGrad}, inOrdinals, true);
  if (bInOrdinalsGrad) runtime("Error: Gradient on inOrdinals is requested, but inOrdinals never has a gradient.");
  std::vector<int64_t> out_sizes;
  const ht_forest_shape s = forest_shape(kind, inData, inThresholds, inOrdinals, inWeights, &outDataGrad, &out_sizes);
  if (size_t(records.numel()) != ht_forest_records_bytes(&s))
    invalid("Error: records do not belong to a forest of this shape.");
  const c10::DeviceGuard guard(inData.device());
  torch::Tensor dx = bInDataGrad ? torch::empty_like(inData) : torch::Tensor();
  torch::Tensor dthr = bInThresholdsGrad ? torch::empty_like(inThresholds) : torch::Tensor();
  torch::Tensor dw = bInWeightsGrad ? torch::empty_like(inWeights) : torch::Tensor();
  const size_t bytes = ht_forest_backward_records_workspace(&s, mode, bInDataGrad, bInThresholdsGrad, bInWeightsGrad);
  torch::Tensor ws = workspace(bytes, inData);
  check(ht_forest_backward_records(&s, ptr(inWeights), ptr(outDataGrad), ptr(records), size_t(records.numel()), ptr(dx),
                                   ptr(dthr), ptr(dw), mode, ptr(ws), bytes, current_stream(inData)));
  return gradient_list(dx, dthr, dw);
}

enum { kLeaf = 0, kMargin = 1, kReach = 2 };

py::object forest_maps(int kind, const torch::Tensor &inData, const torch::Tensor &inThresholds,
                       const torch::Tensor &inOrdinals, const torch::Tensor &inWeights, int want) {
  common_checks({&inData, &inThresholds, &inWeights}, inOrdinals, false);
  std::vector<int64_t> out_sizes;
  const ht_forest_shape s = forest_shape(kind, inData, inThresholds, inOrdinals, inWeights, nullptr, &out_sizes);
  std::vector<int64_t> map_sizes = {inData.size(0), inWeights.size(0)};
  map_sizes.insert(map_sizes.end(), inData.sizes().begin() + 2, inData.sizes().end());
  const c10::DeviceGuard guard(inData.device());
  const auto longs = inData.options().dtype(torch::kInt64);
  torch::Tensor leaf, margins, ordinals, reach;
  if (want == kLeaf) leaf = torch::empty(map_sizes, longs);
  if (want == kMargin) {
    margins = torch::empty(map_sizes, inData.options());
    ordinals = torch::empty(map_sizes, longs);
  }
  if (want == kReach) reach = torch::empty({inWeights.size(0), inWeights.size(1)}, longs);
  // packed vertices for the walk and, for reachability, the leaf keys of its histogram
  const size_t bytes = ht_forest_maps_workspace(&s, want == kReach);
  const torch::Tensor ws = workspace(bytes, inData);
  check(ht_forest_maps(&s, ptr(inData), ptr(inThresholds), static_cast<const int64_t *>(ptr(inOrdinals)),
                       static_cast<int64_t *>(ptr(leaf)), ptr(margins), static_cast<int64_t *>(ptr(ordinals)),
                       static_cast<int64_t *>(ptr(reach)), ptr(ws), bytes, current_stream(inData)));
  if (want == kLeaf) return py::cast(leaf);
  if (want == kReach) return py::cast(reach);
  py::list r;
  r.append(margins);
  r.append(ordinals);
  return r;
}

// hingetree.cpp:930-1076 (dispatch) and :513-581 (shape rules): CPU tensors only, `fix` works in place.
std::vector<bool> thresholds(int kind, bool fix, torch::Tensor inThresholds, const torch::Tensor &inOrdinals,
                             const torch::Tensor &inWeights) {
  if (inOrdinals.scalar_type() != torch::kInt64 || inThresholds.scalar_type() != inWeights.scalar_type())
    invalid("Error: inThresholds, inWeights are expected to share the same torch real number data type. inOrdinals is "
            "expected to be type torch.int64.");
  if (!inThresholds.device().is_cpu() || inOrdinals.device() != inThresholds.device() ||
      inWeights.device() != inThresholds.device())
    invalid("Error: All tensors are expected to be on the CPU.");
  if (!(inThresholds.is_contiguous() && inOrdinals.is_contiguous() && inWeights.is_contiguous()))
    invalid("Error: All tensors are expected to be contiguous.");
  if (inThresholds.scalar_type() != torch::kFloat32 && inThresholds.scalar_type() != torch::kFloat64)
    invalid("Error: Unsupported data type. Only torch.float32 and torch.float64 are supported.");
  if (inThresholds.dim() != 2 || inOrdinals.dim() != 2 || inWeights.dim() < 2)
    invalid("Error: inWeights must have at least 2 dimensions. inThresholds and inOrdinals must have 2 dimensions.");
  if (inThresholds.sizes() != inOrdinals.sizes() || inWeights.size(0) != inThresholds.size(0))
    invalid("Error: inThresholds and inOrdinals must be the same shape. inWeights.shape[0] must be the same as "
            "inThresholds.shape[0].");
  const int64_t depth = compute_depth(inWeights.size(1));
  const int64_t want = depth < 0 ? -1 : (kind == HT_FERN ? depth : (int64_t(1) << depth) - 1);
  if (depth > 31 || depth < 0 || inThresholds.size(1) != want) depth_error(depth);
  const int64_t T = inThresholds.size(0);
  std::vector<uint8_t> flags(size_t(T > 0 ? T : 1));
  if (fix)
    check(ht_fix_thresholds(inThresholds.data_ptr(), static_cast<const int64_t *>(inOrdinals.data_ptr()), T, depth,
                            dtype_code(inThresholds), kind, flags.data()));
  else
    check(ht_check_thresholds(inThresholds.data_ptr(), static_cast<const int64_t *>(inOrdinals.data_ptr()), T, depth,
                              dtype_code(inThresholds), kind, flags.data()));
  std::vector<bool> r;
  for (int64_t i = 0; i < T; ++i) r.push_back(flags[size_t(i)] != 0);
  return r;
}

// ---- convolution ------------------------------------------------------------------------------------------------
// Rules of hingetree_conv_cpu_forward / _backward (hingetree_conv.cpp:58-122,240-332).
ht_conv_shape conv_shape(int kind, int nd, const torch::Tensor &inData, const torch::Tensor &inThresholds,
                         const torch::Tensor &inOrdinals, const torch::Tensor &inWeights,
                         const std::vector<int64_t> &kernelSize, const std::vector<int64_t> &stride,
                         const std::vector<int64_t> &padding, const std::vector<int64_t> &dilation,
                         const torch::Tensor *outDataGrad, std::vector<int64_t> *out_sizes) {
  const std::string nds = std::to_string(nd);
  if (int(kernelSize.size()) != nd || int(stride.size()) != nd || int(padding.size()) != nd || int(dilation.size()) != nd)
    invalid("Error: kernel, stride, padding, dilation all expected to have " + nds + " dimensions.");
  if (inData.dim() != nd + 2 || inThresholds.dim() != 3 || inOrdinals.dim() != 3 || inWeights.dim() < 3)
    invalid("Error: inData expected to have " + std::to_string(nd + 2) +
            " dimensions. inThresholds, inOrdinals expected to have 3 dimensions. inWeights expected to be less than 3 "
            "dimensions.");
  if (inThresholds.sizes() != inOrdinals.sizes() || inWeights.size(0) != inThresholds.size(0))
    invalid("Error: inThresholds and inOrdinals must be the same shape. inWeights.shape[0] must be the same as "
            "inThresholds.shape[0].");
  if (inWeights.size(1) == 0) invalid("Error: inWeights.shape[1] is expected to divide inData.shape[1].");
  const int64_t groups = inData.size(1) / inWeights.size(1);
  if (groups * inWeights.size(1) != inData.size(1))
    invalid("Error: inWeights.shape[1] is expected to divide inData.shape[1].");
  if (groups == 0 || inWeights.size(0) % groups != 0)
    invalid("inData.shape[1]//inWeights.shape[1] is expected to divide output channels.");
  if (groups != 1 || inThresholds.size(1) != inData.size(1))
    // the reference indexes grouped convolutions inconsistently (hingetree_conv.cpp:125 vs :202-206), so only
    // groups == 1 has a defined result
    runtime("Error: grouped hinge tree convolution (inData.shape[1] != inWeights.shape[1]) is not supported.");
  ht_conv_shape s{};
  s.B = inData.size(0);
  s.C = inData.size(1);
  s.Cout = inWeights.size(0);
  s.M = prod(inWeights.sizes(), 3);
  s.dtype = dtype_code(inData);
  s.kind = kind;
  s.nd = nd;
  int64_t taps = 1;
  for (int d = 0; d < nd; ++d) {
    s.size[d] = inData.size(2 + d);
    s.kernel[d] = kernelSize[size_t(d)];
    s.stride[d] = stride[size_t(d)];
    s.padding[d] = padding[size_t(d)];
    s.dilation[d] = dilation[size_t(d)];
    taps *= kernelSize[size_t(d)];
  }
  const int64_t depth = compute_depth(inWeights.size(2));
  s.depth = depth > 0 ? depth : 0;
  int64_t osz[HT_MAX_CONV_DIMS] = {0, 0, 0};
  check(ht_conv_output_size(&s, osz));  // "Unable to convert image patches to matrix."
  require_gpu(inData);
  validate_ordinals(inOrdinals, taps);
  const int64_t want = depth < 0 ? -1 : (kind == HT_FERN ? depth : (int64_t(1) << depth) - 1);
  if (depth > 31 || depth < 0 || inThresholds.size(2) != want) depth_error(depth);
  out_sizes->assign({inData.size(0), inWeights.size(0)});
  for (int d = 0; d < nd; ++d) out_sizes->push_back(osz[d]);
  out_sizes->insert(out_sizes->end(), inWeights.sizes().begin() + 3, inWeights.sizes().end());
  if (outDataGrad && outDataGrad->sizes() != c10::IntArrayRef(*out_sizes))
    invalid("Error: outDataGrad.shape does not match the expected shape (" + sizes_text(outDataGrad->sizes()) +
            " != " + sizes_text(*out_sizes) + ").");
  return s;
}

torch::Tensor conv_forward(int kind, int nd, const torch::Tensor &inData, const torch::Tensor &inThresholds,
                           const torch::Tensor &inOrdinals, const torch::Tensor &inWeights,
                           const std::vector<int64_t> &kernelSize, const std::vector<int64_t> &stride,
                           const std::vector<int64_t> &padding, const std::vector<int64_t> &dilation) {
  common_checks({&inData, &inThresholds, &inWeights}, inOrdinals, false);
  std::vector<int64_t> out_sizes;
  const ht_conv_shape s = conv_shape(kind, nd, inData, inThresholds, inOrdinals, inWeights, kernelSize, stride, padding,
                                     dilation, nullptr, &out_sizes);
  const c10::DeviceGuard guard(inData.device());
  torch::Tensor out = torch::empty(out_sizes, inData.options());
  check(ht_conv_forward(&s, ptr(inData), ptr(inThresholds), static_cast<const int64_t *>(ptr(inOrdinals)),
                        ptr(inWeights), ptr(out), current_stream(inData)));
  return out;
}

py::list conv_backward(int kind, int nd, const torch::Tensor &inData, bool bInDataGrad,
                       const torch::Tensor &inThresholds, bool bInThresholdsGrad, const torch::Tensor &inOrdinals,
                       bool bInOrdinalsGrad, const torch::Tensor &inWeights, bool bInWeightsGrad,
                       const torch::Tensor &outDataGrad, const std::vector<int64_t> &kernelSize,
                       const std::vector<int64_t> &stride, const std::vector<int64_t> &padding,
                       const std::vector<int64_t> &dilation) {
  common_checks({&inData, &inThresholds, &inWeights, &outDataGrad}, inOrdinals, true);
  if (bInOrdinalsGrad)  // hingetree_conv.cpp:235-238
    runtime("Error: Gradient on inOrdinals is requested, but inOrdinals never has a gradient.");
  std::vector<int64_t> out_sizes;
  const ht_conv_shape s = conv_shape(kind, nd, inData, inThresholds, inOrdinals, inWeights, kernelSize, stride, padding,
                                     dilation, &outDataGrad, &out_sizes);
  const c10::DeviceGuard guard(inData.device());
  torch::Tensor dx = bInDataGrad ? torch::empty_like(inData) : torch::Tensor();
  torch::Tensor dthr = bInThresholdsGrad ? torch::empty_like(inThresholds) : torch::Tensor();
  torch::Tensor dw = bInWeightsGrad ? torch::empty_like(inWeights) : torch::Tensor();
  check(ht_conv_backward(&s, ptr(inData), ptr(inThresholds), static_cast<const int64_t *>(ptr(inOrdinals)),
                         ptr(inWeights), ptr(outDataGrad), ptr(dx), ptr(dthr), ptr(dw), current_stream(inData)));
  return gradient_list(dx, dthr, dw);
}

}  // namespace

// The reference's names and positional signatures (hingetree.cpp:1963-2003) for the path this build serves, plus the
// kind-parametrised entries the Python operator layer builds its other operators on. Operators outside the path are
// not defined here (the Python layer's stubs raise for them).
PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "native host of hingetree_cpp (forest / fern / convolution path) over libhingetree_hip.so";
  m.attr("abi_version") = HT_ABI_VERSION;  // of the header this module was compiled against, not of the loaded library
  m.def("forget_ordinal_checks", &forget_ordinal_checks);

  m.def("forest_forward", &forest_forward);
  m.def("forest_backward", &forest_backward);
  m.def("forest_forward_records", &forest_forward_records);
  m.def("forest_backward_records", &forest_backward_records);
  m.def("forest_maps", &forest_maps);
  m.def("forest_thresholds", &thresholds);
  m.def("conv_forward", &conv_forward);
  m.def("conv_backward", &conv_backward);

#define HT_FOREST_OPS(prefix, KIND)                                                                                   \
  m.def(prefix "_forward", [](const torch::Tensor &x, const torch::Tensor &thr, const torch::Tensor &ord,             \
                              const torch::Tensor &w) { return forest_forward(KIND, x, thr, ord, w); });              \
  m.def(prefix "_backward",                                                                                           \
        [](const torch::Tensor &x, bool bx, const torch::Tensor &thr, bool bthr, const torch::Tensor &ord, bool bord,  \
           const torch::Tensor &w, bool bw, const torch::Tensor &g) {                                                 \
          return forest_backward(KIND, HT_BACKWARD_ATOMIC, x, bx, thr, bthr, ord, bord, w, bw, g);                    \
        });                                                                                                           \
  m.def(prefix "_backward_deterministic",                                                                             \
        [](const torch::Tensor &x, bool bx, const torch::Tensor &thr, bool bthr, const torch::Tensor &ord, bool bord,  \
           const torch::Tensor &w, bool bw, const torch::Tensor &g) {                                                 \
          return forest_backward(KIND, HT_BACKWARD_DETERMINISTIC, x, bx, thr, bthr, ord, bord, w, bw, g);             \
        });                                                                                                           \
  m.def(prefix "_forward_records", [](const torch::Tensor &x, const torch::Tensor &thr, const torch::Tensor &ord,     \
                                      const torch::Tensor &w) { return forest_forward_records(KIND, x, thr, ord, w); }); \
  m.def(prefix "_backward_records",                                                                                   \
        [](const torch::Tensor &records, bool deterministic, const torch::Tensor &x, bool bx, const torch::Tensor &thr, \
           bool bthr, const torch::Tensor &ord, bool bord, const torch::Tensor &w, bool bw, const torch::Tensor &g) {  \
          return forest_backward_records(KIND, deterministic ? HT_BACKWARD_DETERMINISTIC : HT_BACKWARD_ATOMIC,        \
                                         records, x, bx, thr, bthr, ord, bord, w, bw, g);                             \
        });                                                                                                           \
  m.def(prefix "_leafmap", [](const torch::Tensor &x, const torch::Tensor &thr, const torch::Tensor &ord,             \
                              const torch::Tensor &w) { return forest_maps(KIND, x, thr, ord, w, kLeaf); });          \
  m.def(prefix "_marginmap", [](const torch::Tensor &x, const torch::Tensor &thr, const torch::Tensor &ord,           \
                                const torch::Tensor &w) { return forest_maps(KIND, x, thr, ord, w, kMargin); });      \
  m.def(prefix "_reachability", [](const torch::Tensor &x, const torch::Tensor &thr, const torch::Tensor &ord,        \
                                   const torch::Tensor &w) { return forest_maps(KIND, x, thr, ord, w, kReach); });    \
  m.def(prefix "_check_thresholds", [](const torch::Tensor &thr, const torch::Tensor &ord, const torch::Tensor &w) {  \
    return thresholds(KIND, false, thr, ord, w);                                                                      \
  });                                                                                                                 \
  m.def(prefix "_fix_thresholds", [](const torch::Tensor &thr, const torch::Tensor &ord, const torch::Tensor &w) {    \
    return thresholds(KIND, true, thr, ord, w);                                                                       \
  });
  HT_FOREST_OPS("tree", HT_TREE)
  HT_FOREST_OPS("fern", HT_FERN)
#undef HT_FOREST_OPS

#define HT_CONV_OPS(prefix, KIND, ND)                                                                                 \
  m.def(prefix "_forward",                                                                                            \
        [](const torch::Tensor &x, const torch::Tensor &thr, const torch::Tensor &ord, const torch::Tensor &w,        \
           const std::vector<int64_t> &k, const std::vector<int64_t> &s, const std::vector<int64_t> &p,               \
           const std::vector<int64_t> &d) { return conv_forward(KIND, ND, x, thr, ord, w, k, s, p, d); });            \
  m.def(prefix "_backward",                                                                                           \
        [](const torch::Tensor &x, bool bx, const torch::Tensor &thr, bool bthr, const torch::Tensor &ord, bool bord,  \
           const torch::Tensor &w, bool bw, const torch::Tensor &g, const std::vector<int64_t> &k,                    \
           const std::vector<int64_t> &s, const std::vector<int64_t> &p, const std::vector<int64_t> &d) {             \
          return conv_backward(KIND, ND, x, bx, thr, bthr, ord, bord, w, bw, g, k, s, p, d);                          \
        });
  HT_CONV_OPS("tree_conv1d", HT_TREE, 1)
  HT_CONV_OPS("tree_conv2d", HT_TREE, 2)
  HT_CONV_OPS("tree_conv3d", HT_TREE, 3)
  HT_CONV_OPS("fern_conv1d", HT_FERN, 1)
  HT_CONV_OPS("fern_conv2d", HT_FERN, 2)
  HT_CONV_OPS("fern_conv3d", HT_FERN, 3)
#undef HT_CONV_OPS
}
